// The weight update pass of the C++ poplin layer: calculateWeightDeltas,
// convolutionWeightUpdate, convolutionBiasUpdate over the C ABI.
#include "LayerInternal.hpp"
#include "poplin/ConvUtil.hpp"
#include "poplin/Convolution.hpp"
#include "poputil/exceptions.hpp"

#include <ostream>

namespace poplin {

using namespace detail;

namespace {

/// getWeightUpdateOptions (lib/poplin/ConvUtilInternal.cpp:941-954) on
/// option flags: only `pass` changes.
poplar::OptionFlags weightUpdateOptions(const poplar::OptionFlags &fwd) {
  poplar::OptionFlags wu = fwd;
  std::string pass = "NONE";
  for (const auto &kv : fwd)
    if (kv.first == "pass")
      pass = kv.second;
  wu.set("pass",
         pass.rfind("FC_", 0) == 0 ? "FC_TRAINING_WU" : "TRAINING_WU");
  return wu;
}

std::vector<std::size_t> weightsShape(const ConvParams &p) {
  std::vector<std::size_t> shape{p.numConvGroups, p.outputChannelsPerConvGroup,
                                 p.inputChannelsPerConvGroup};
  shape.insert(shape.end(), p.kernelShape.begin(), p.kernelShape.end());
  return shape;
}

std::vector<std::size_t> actsShape(std::size_t batch, std::size_t chans,
                                   const std::vector<std::size_t> &field) {
  std::vector<std::size_t> shape{batch, chans};
  shape.insert(shape.end(), field.begin(), field.end());
  return shape;
}

/// `t` held channels-last.  The forward input may also arrive in the
/// external layout: it is converted with the forward plan's layout kernel.
DeviceTensor channelsLast(const DeviceTensor &t, const char *what,
                          const std::vector<std::size_t> &expectedShape,
                          const PlanHandle *fwdPlanOfInput, Stream &prog) {
  if (t.shape() != expectedShape)
    throw poputil::poplibs_error(std::string(what) +
                                 " does not have the shape the convolution "
                                 "parameters give");
  if (t.layout() == DeviceTensor::Layout::ChannelsLast)
    return t;
  if (t.layout() != DeviceTensor::Layout::External || !fwdPlanOfInput)
    throw poputil::poplibs_error(
        std::string(what) + " must be held channels-last (convolution results "
                            "and createConvOutput tensors are)");
  DeviceTensor cl(t.elementType(), t.shape(),
                  DeviceTensor::Layout::ChannelsLast, t.bytes());
  check(mxconv_acts_to_internal(fwdPlanOfInput->plan, t.data(), cl.data(),
                                streamOf(prog)));
  return cl;
}

struct Operands {
  DeviceTensor zDeltas, activations;
  std::shared_ptr<PlanHandle> plan;
  DeviceTensor workspace;
  std::size_t workspaceBytes = 0;
};

Operands prepare(const DeviceTensor &zDeltas, const DeviceTensor &activations,
                 const ConvParams &params, Stream &prog,
                 const poplar::OptionFlags &options, PlanningCache *cache) {
  if (zDeltas.elementType() != params.inputType ||
      activations.elementType() != params.inputType)
    throw poputil::poplibs_error(
        "The deltas and activations of the weight update pass have the "
        "convolution's input type");
  Operands o;
  const auto fwdPlan = getPlan(params, options, cache);
  o.activations = channelsLast(
      activations, "activations",
      actsShape(params.batchSize, params.getNumInputChans(),
                params.inputFieldShape),
      fwdPlan.get(), prog);
  o.zDeltas = channelsLast(zDeltas, "zDeltas",
                           actsShape(params.batchSize,
                                     params.getNumOutputChans(),
                                     params.getOutputFieldShape()),
                           nullptr, prog);
  o.plan = getPlan(getWeightUpdateParams(params), weightUpdateOptions(options),
                   cache);
  check(mxconv_weight_update_workspace_bytes(o.plan->plan, &o.workspaceBytes));
  o.workspace = DeviceTensor(poplar::FLOAT, {o.workspaceBytes / 4 + 1},
                             DeviceTensor::Layout::External,
                             o.workspaceBytes + 4);
  return o;
}

} // namespace

std::uint64_t getBwdFlops(const ConvParams &params) {
  return getFwdFlops(params);
}
std::uint64_t getWuFlops(const ConvParams &params) {
  return getFwdFlops(params);
}

DeviceTensor calculateWeightDeltas(const DeviceTensor &zDeltas,
                                   const DeviceTensor &activations,
                                   const ConvParams &params, Stream &prog,
                                   const poplar::OptionFlags &options,
                                   PlanningCache *cache) {
  const Operands o = prepare(zDeltas, activations, params, prog, options, cache);
  const auto shape = weightsShape(params);
  std::size_t elems = 1;
  for (auto s : shape)
    elems *= s;
  DeviceTensor deltas(params.outputType, shape, DeviceTensor::Layout::External,
                      elems * params.outputType.size());
  check(mxconv_calculate_weight_deltas(
      o.plan->plan, o.zDeltas.data(), o.activations.data(), deltas.data(),
      o.workspace.data(), o.workspaceBytes, streamOf(prog)));
  prog.synchronize(); // the workspace is released on return
  return deltas;
}

void convolutionWeightUpdate(const DeviceTensor &zDeltas,
                             const DeviceTensor &weights,
                             const DeviceTensor &activations,
                             ConvParams params, float scale, Stream &prog,
                             const poplar::OptionFlags &options,
                             PlanningCache *cache) {
  // The deltas are formed in the weights' type
  // (lib/poplin/Convolution.cpp:3533-3535).
  params.outputType = params.inputType;
  if (weights.shape() != weightsShape(params) ||
      weights.elementType() != params.inputType)
    throw poputil::poplibs_error(
        "The weights do not have the shape and type the convolution "
        "parameters give");
  const Operands o = prepare(zDeltas, activations, params, prog, options, cache);
  if (weights.layout() == DeviceTensor::Layout::External) {
    check(mxconv_convolution_weight_update(
        o.plan->plan, o.zDeltas.data(), weights.data(), o.activations.data(),
        scale, o.workspace.data(), o.workspaceBytes, streamOf(prog)));
    prog.synchronize();
    return;
  }
  if (weights.layout() != DeviceTensor::Layout::PackedWeights ||
      !weights.packedFor)
    throw poputil::poplibs_error(
        "convolutionWeightUpdate takes weights in the external layout or as "
        "createWeights made them");
  // Packing only moves elements and fills the gaps with zeros, so the update
  // can be applied in the packing: pack the deltas the same way and add.
  const auto *packing = static_cast<const PlanHandle *>(weights.packedFor.get());
  DeviceTensor deltas(params.inputType, weights.shape(),
                      DeviceTensor::Layout::External,
                      weights.numElements() * params.inputType.size());
  check(mxconv_calculate_weight_deltas(
      o.plan->plan, o.zDeltas.data(), o.activations.data(), deltas.data(),
      o.workspace.data(), o.workspaceBytes, streamOf(prog)));
  const std::size_t packedBytes =
      bufferBytes(packing->plan, MXCONV_BUFFER_WEIGHTS_PACKED);
  if (packedBytes != weights.bytes())
    throw poputil::poplibs_error("The weights' packing does not match their "
                                 "size");
  DeviceTensor packedDeltas(params.inputType, weights.shape(),
                            DeviceTensor::Layout::PackedWeights, packedBytes);
  check(mxconv_pack_weights(packing->plan, deltas.data(), packedDeltas.data(),
                            streamOf(prog)));
  check(mxconv_scaled_add_to(params.inputType.id(), weights.data(), 1.f,
                             packedDeltas.data(), scale,
                             packedBytes / params.inputType.size(),
                             streamOf(prog)));
  prog.synchronize();
}

void convolutionBiasUpdate(const DeviceTensor &zDeltas,
                           const DeviceTensor &biases, float scale,
                           const poplar::OptionFlags &options, Stream &prog) {
  convolutionValidateOptions(options);
  if (zDeltas.shape().size() < 2)
    throw poputil::poplibs_error(
        "convolutionBiasUpdate with rank " +
        std::to_string(zDeltas.shape().size()) +
        "; must have at least channel and batch dimensions");
  if (zDeltas.layout() != DeviceTensor::Layout::ChannelsLast)
    throw poputil::poplibs_error(
        "convolutionBiasUpdate: zDeltas must be held channels-last "
        "(convolution results and createConvOutput tensors are)");
  const std::size_t chans = zDeltas.shape()[1];
  if (biases.shape() != std::vector<std::size_t>{chans} ||
      biases.layout() != DeviceTensor::Layout::External)
    throw poputil::poplibs_error(
        "convolutionBiasUpdate: one bias per channel is needed");
  const std::size_t outer = chans ? zDeltas.numElements() / chans : 0;
  std::size_t wsBytes = 0;
  check(mxconv_bias_update_workspace_bytes(outer, chans, &wsBytes));
  DeviceTensor workspace(poplar::FLOAT, {wsBytes / 4 + 1},
                         DeviceTensor::Layout::External, wsBytes + 4);
  check(mxconv_convolution_bias_update(
      zDeltas.elementType().id(), zDeltas.data(), outer, chans,
      biases.elementType().id(), biases.data(), scale, workspace.data(),
      wsBytes, streamOf(prog)));
  prog.synchronize(); // the workspace is released on return
}

void reportWeightUpdatePlanInfo(std::ostream &out, const ConvParams &fwdParams,
                                const poplar::OptionFlags &fwdOptions,
                                PlanningCache *cache) {
  reportPlanInfo(out, getWeightUpdateParams(fwdParams),
                 weightUpdateOptions(fwdOptions), cache);
}

} // namespace poplin

// poplin::multiconv over the C ABI: operands are brought into the device
// layouts, then every forward pass goes to the device in one
// mxconv_multi_fwd call, which fuses what it can into shared launches.
#include "poplin/MultiConvolution.hpp"
#include "LayerInternal.hpp"
#include "poputil/exceptions.hpp"

namespace poplin {
namespace multiconv {

using namespace detail;

namespace {

/// True for planType parallel (the default); throws on a bad option.
bool parallelPlan(const poplar::OptionFlags &options) {
  std::vector<const char *> keys, values;
  for (const auto &kv : options) {
    keys.push_back(kv.first.c_str());
    values.push_back(kv.second.c_str());
  }
  int parallel = 1;
  check(mxconv_multiconv_validate_options(keys.data(), values.data(),
                                          keys.size(), &parallel));
  return parallel != 0;
}

/// The convolutions of a parallel plan share one lowering in PopLibs, so
/// their `insertTransformsCycleCountProgs` options must agree
/// (lib/poplin/MultiConvolution.cpp:155-173).  The option itself has no
/// effect on this device; the error is kept.
template <class Args> void requireSameCycleCountProgs(const Args &args) {
  auto wanted = [](const poplar::OptionFlags &options) {
    for (const auto &kv : options)
      if (kv.first == "insertTransformsCycleCountProgs")
        return kv.second == "true";
    return false;
  };
  for (const auto &arg : args)
    if (wanted(arg.options) != wanted(args.front().options))
      throw poputil::poplibs_error(
          "Parallel multi-plans require to have same value for "
          "<insertTransformsCycleCountProgs> option");
}

std::vector<std::size_t> actsShape(std::size_t batch, std::size_t chans,
                                   const std::vector<std::size_t> &field) {
  std::vector<std::size_t> shape{batch, chans};
  shape.insert(shape.end(), field.begin(), field.end());
  return shape;
}

} // namespace

void validateOptions(const poplar::OptionFlags &options) {
  parallelPlan(options);
}

DeviceTensor createWeights(const std::vector<CreateTensorArgs> &args,
                           unsigned weightsIndex,
                           const poplar::OptionFlags &options,
                           PlanningCache *cache) {
  parallelPlan(options);
  const auto &arg = args.at(weightsIndex);
  return poplin::createWeights(arg.params, arg.options, cache);
}

DeviceTensor createInput(const std::vector<CreateTensorArgs> &args,
                         unsigned inputIndex,
                         const poplar::OptionFlags &options,
                         PlanningCache *cache) {
  parallelPlan(options);
  const auto &arg = args.at(inputIndex);
  return poplin::createInput(arg.params, arg.options, cache);
}

void weightsTransposeChansFlipXY(std::vector<ConvolutionArgs> &args,
                                 const std::vector<DeviceTensor> &weightsIn,
                                 Stream &prog,
                                 const poplar::OptionFlags &options,
                                 PlanningCache *) {
  parallelPlan(options);
  if (args.size() != weightsIn.size())
    throw poputil::poplibs_error(
        "multiconv::weightsTransposeChansFlipXY: one weights tensor per "
        "convolution is needed");
  for (std::size_t i = 0; i != args.size(); ++i)
    poplin::weightsTransposeChansFlipXY(weightsIn[i], args[i].weights, prog);
}

std::vector<DeviceTensor> convolution(const std::vector<ConvolutionArgs> &args,
                                      bool transposeAndFlipWeights,
                                      Stream &prog,
                                      const poplar::OptionFlags &options,
                                      PlanningCache *cache) {
  const bool parallel = parallelPlan(options);
  if (parallel)
    requireSameCycleCountProgs(args);
  const std::size_t n = args.size();
  std::vector<std::shared_ptr<PlanHandle>> plans(n);
  std::vector<DeviceTensor> in(n), weights(n), out(n), workspace(n);
  std::vector<const mxconv_plan *> planPtrs(n);
  std::vector<const void *> inPtrs(n), weightPtrs(n);
  std::vector<void *> outPtrs(n), workspacePtrs(n);
  std::vector<std::size_t> workspaceBytes(n);
  std::vector<std::uint8_t> inMeta(n), weightMeta(n);
  bool temporaries = false;
  for (std::size_t i = 0; i != n; ++i) {
    const auto &arg = args[i];
    const ConvParams &p = arg.params;
    plans[i] = getPlan(p, arg.options, cache);
    const mxconv_plan *plan = plans[i]->plan;
    if (arg.inputs.shape() !=
        actsShape(p.batchSize, p.getNumInputChans(), p.inputFieldShape))
      throw poputil::poplibs_error(
          "multiconv::convolution: input " + std::to_string(i) +
          " does not have the shape its parameters give");
    // Operands in the external layout are converted on the caller's stream,
    // as the single-convolution entry point does.
    in[i] = arg.inputs;
    if (arg.inputs.layout() == DeviceTensor::Layout::External) {
      in[i] = DeviceTensor(arg.inputs.elementType(), arg.inputs.shape(),
                           DeviceTensor::Layout::ChannelsLast,
                           arg.inputs.bytes());
      check(mxconv_acts_to_internal(plan, arg.inputs.data(), in[i].data(),
                                    streamOf(prog)));
      temporaries = true;
    }
    weights[i] = arg.weights;
    if (transposeAndFlipWeights) {
      if (arg.weights.layout() != DeviceTensor::Layout::External)
        throw poputil::poplibs_error(
            "multiconv::convolution: transposeAndFlipWeights takes the "
            "forward weights in the external layout");
      std::vector<std::size_t> flippedShape = arg.weights.shape();
      if (flippedShape.size() < 3)
        throw poputil::poplibs_error("multiconv::convolution: bad weights");
      std::swap(flippedShape[1], flippedShape[2]);
      DeviceTensor flipped(arg.weights.elementType(), flippedShape,
                           DeviceTensor::Layout::External,
                           arg.weights.bytes());
      flipped.metadata = arg.weights.metadata;
      poplin::weightsTransposeChansFlipXY(arg.weights, flipped, prog);
      weights[i] = flipped;
      temporaries = true;
    }
    if (weights[i].layout() == DeviceTensor::Layout::PackedWeights)
      requirePackedFor(plan, weights[i], "weights");
    if (weights[i].layout() == DeviceTensor::Layout::External) {
      DeviceTensor packed(weights[i].elementType(), weights[i].shape(),
                          DeviceTensor::Layout::PackedWeights,
                          bufferBytes(plan, MXCONV_BUFFER_WEIGHTS_PACKED));
      packed.metadata = weights[i].metadata;
      check(mxconv_pack_weights(plan, weights[i].data(), packed.data(),
                                streamOf(prog)));
      weights[i] = packed;
      temporaries = true;
    }
    out[i] = poplin::createConvOutput(p, arg.options, cache);
    workspaceBytes[i] = bufferBytes(plan, MXCONV_BUFFER_WORKSPACE);
    if (workspaceBytes[i]) {
      workspace[i] = DeviceTensor(poplar::FLOAT, {workspaceBytes[i] / 4},
                                  DeviceTensor::Layout::External,
                                  workspaceBytes[i]);
      temporaries = true;
    }
    planPtrs[i] = plan;
    inPtrs[i] = in[i].data();
    weightPtrs[i] = weights[i].data();
    outPtrs[i] = out[i].data();
    workspacePtrs[i] = workspace[i].data();
    inMeta[i] = arg.inputs.metadata.byte();
    weightMeta[i] = arg.weights.metadata.byte();
  }
  check(mxconv_multi_fwd(n, planPtrs.data(), inPtrs.data(), inMeta.data(),
                         weightPtrs.data(), weightMeta.data(), nullptr,
                         outPtrs.data(), workspacePtrs.data(),
                         workspaceBytes.data(), parallel ? 1 : 0,
                         streamOf(prog)));
  if (temporaries)
    prog.synchronize(); // they are released on return
  return out;
}

std::vector<DeviceTensor>
calculateWeightDeltas(const std::vector<CalculateWeightDeltasArgs> &args,
                      Stream &prog, const poplar::OptionFlags &options,
                      PlanningCache *cache) {
  // PopLibs implements this for serial plans only
  // (lib/poplin/MultiConvolution.cpp:317-333); the passes run one after
  // another here whatever the plan type.
  parallelPlan(options);
  std::vector<DeviceTensor> deltas;
  deltas.reserve(args.size());
  for (const auto &arg : args)
    deltas.push_back(poplin::calculateWeightDeltas(
        arg.zDeltas, arg.activations, arg.params, prog, arg.options, cache));
  return deltas;
}

void convolutionWeightUpdate(const std::vector<ConvWeightUpdateArgsScalar> &args,
                             Stream &prog, const poplar::OptionFlags &options,
                             PlanningCache *cache) {
  parallelPlan(options);
  for (const auto &arg : args) {
    // lib/poplin/MultiConvolution.cpp:360-366
    if (arg.params.inputType != arg.params.outputType)
      throw poputil::poplibs_error(
          "multiconv::convolutionWeightUpdate does not support having a "
          "different input and output type.");
    poplin::convolutionWeightUpdate(arg.zDeltas, arg.weights, arg.activations,
                                    arg.params, arg.scale, prog, arg.options,
                                    cache);
  }
}

} // namespace multiconv
} // namespace poplin

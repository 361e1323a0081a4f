// The C++ poplin entry points, written over the C ABI of mxconv.h.  Device
// memory and host transfers use the HIP runtime directly; every kernel launch
// goes through an mxconv_* call.
#include "poplin/Convolution.hpp"
#include "poplin/ConvPreplan.hpp"
#include "LayerInternal.hpp"
#include "mxconv.h"
#include "poplar/exceptions.hpp"
#include "poputil/exceptions.hpp"

#include <algorithm>
#include <atomic>
#include <exception>
#include <set>
#include <thread>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <ostream>
#include <string>
#include <tuple>

namespace poplin {

namespace detail {

[[noreturn]] static void raise(mxconv_status s) {
  const std::string message = mxconv_last_error();
  switch (s) {
  case MXCONV_INVALID_OPTION:
    throw poplar::invalid_option(message);
  case MXCONV_OUT_OF_MEMORY:
    throw poplar::graph_memory_allocation_error(message);
  default:
    throw poputil::poplibs_error(message.empty() ? mxconv_status_string(s)
                                                 : message);
  }
}
void check(mxconv_status s) {
  if (s != MXCONV_OK)
    raise(s);
}
static void checkHip(hipError_t e, const char *what) {
  if (e == hipSuccess)
    return;
  const std::string message = std::string(what) + ": " + hipGetErrorString(e);
  if (e == hipErrorOutOfMemory)
    throw poplar::graph_memory_allocation_error(message);
  throw poputil::poplibs_error(message);
}

static std::shared_ptr<PlanHandle> createPlan(const ConvParams &params,
                                       const poplar::OptionFlags &options) {
  mxconv_params c;
  params.toC(c);
  std::vector<const char *> keys, values;
  for (const auto &kv : options) {
    keys.push_back(kv.first.c_str());
    values.push_back(kv.second.c_str());
  }
  mxconv_plan *plan = nullptr;
  check(mxconv_plan_create(&c, keys.data(), values.data(), keys.size(), &plan));
  return std::make_shared<PlanHandle>(plan);
}

std::size_t bufferBytes(const mxconv_plan *plan, mxconv_buffer which) {
  std::size_t bytes = 0;
  check(mxconv_plan_buffer_bytes(plan, which, &bytes));
  return bytes;
}

void requirePackedFor(const mxconv_plan *plan, const DeviceTensor &packed,
                      const char *what) {
  const auto *packing = static_cast<const PlanHandle *>(packed.packedFor.get());
  int32_t same = 0;
  if (packing)
    check(mxconv_plans_pack_alike(plan, packing->plan, &same));
  if (!same)
    throw poputil::poplibs_error(
        std::string("The ") + what +
        " were arranged (createWeights, preArrangeMatMulInputRHS) for another "
        "plan than the one these parameters and options give: pass them in "
        "the external layout or create them with the same options");
}

static std::vector<std::size_t> actsShape(std::size_t batch, std::size_t chans,
                                   const std::vector<std::size_t> &field) {
  std::vector<std::size_t> shape{batch, chans};
  shape.insert(shape.end(), field.begin(), field.end());
  return shape;
}

mxconv_stream streamOf(const Stream &s) {
  return static_cast<mxconv_stream>(s.handle());
}

} // namespace detail
using namespace detail;

// ---- Stream ---------------------------------------------------------------

struct Stream::Impl {
  hipStream_t stream = nullptr;
  bool owned = false;
  ~Impl() {
    if (owned && stream)
      (void)hipStreamDestroy(stream);
  }
};

Stream::Stream() : impl_(std::make_shared<Impl>()) {
  checkHip(hipStreamCreate(&impl_->stream), "hipStreamCreate");
  impl_->owned = true;
}
Stream::Stream(void *hipStream) : impl_(std::make_shared<Impl>()) {
  impl_->stream = static_cast<hipStream_t>(hipStream);
}
void *Stream::handle() const { return impl_->stream; }
void Stream::synchronize() const {
  checkHip(hipStreamSynchronize(impl_->stream), "hipStreamSynchronize");
}

// ---- DeviceTensor ---------------------------------------------------------

DeviceTensor::DeviceTensor(poplar::Type type, std::vector<std::size_t> shape,
                           Layout layout, std::size_t bytes)
    : type_(type), shape_(std::move(shape)), layout_(layout), bytes_(bytes) {
  void *p = nullptr;
  // A zero-sized tensor still gets a distinct, valid allocation.
  checkHip(hipMalloc(&p, bytes ? bytes : 1), "hipMalloc");
  buffer_ = std::shared_ptr<void>(p, [](void *q) { (void)hipFree(q); });
}

std::size_t DeviceTensor::numElements() const {
  std::size_t n = 1;
  for (auto s : shape_)
    n *= s;
  return n;
}

// ---- PlanningCache --------------------------------------------------------

struct PlanningCache::Impl {
  using Key = std::pair<ConvParams, poplar::OptionFlags>;
  std::mutex mutex;
  std::map<Key, std::shared_ptr<PlanHandle>> plans;
};
PlanningCache::PlanningCache() : impl(new Impl) {}
PlanningCache::~PlanningCache() = default;
std::size_t PlanningCache::size() const {
  std::lock_guard<std::mutex> lock(impl->mutex);
  return impl->plans.size();
}

namespace detail {
std::shared_ptr<PlanHandle> getPlan(const ConvParams &params,
                                    const poplar::OptionFlags &options,
                                    PlanningCache *cache) {
  if (!cache)
    return createPlan(params, options);
  // Plans are keyed by the canonical parameters, as in PopLibs, so that
  // descriptors which differ only in unused padding share a plan.  The
  // caller-visible tensor shapes are identical for both.
  const PlanningCache::Impl::Key key{params.canonicalize(), options};
  std::lock_guard<std::mutex> lock(cache->impl->mutex);
  auto it = cache->impl->plans.find(key);
  if (it != cache->impl->plans.end())
    return it->second;
  auto plan = createPlan(params, options);
  cache->impl->plans.emplace(key, plan);
  return plan;
}
} // namespace detail

// ---- entry points ---------------------------------------------------------

std::uint64_t getFwdFlops(const ConvParams &params) {
  mxconv_params c;
  params.toC(c);
  std::uint64_t flops = 0;
  check(mxconv_get_fwd_flops(&c, &flops));
  return flops;
}

namespace {
double perfectCycleCount(const ConvParams &params) {
  // Dense MFMA, MACs per cycle and SIMD: 16x16x32 fp16 in 16 cycles,
  // 16x16x128 fp8 in 32, 32x32x2 fp32 in 64.
  const double perSimd = params.inputType == poplar::FLOAT     ? 32.0
                         : params.inputType == poplar::QUARTER ? 1024.0
                                                               : 512.0;
  const double perChip = perSimd * 4 * poplar::Target::gfx950().getNumComputeUnits();
  return double(getFwdFlops(params) / 2) / perChip;
}
} // namespace

double getFwdPerfectCycleCount(const ConvParams &params) {
  return perfectCycleCount(params);
}
double getBwdPerfectCycleCount(const ConvParams &params) {
  return perfectCycleCount(params);
}
double getWuPerfectCycleCount(const ConvParams &params) {
  return perfectCycleCount(params);
}

DeviceTensor createWeights(const ConvParams &params,
                           const poplar::OptionFlags &options,
                           PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  std::vector<std::size_t> shape{params.numConvGroups,
                                 params.outputChannelsPerConvGroup,
                                 params.inputChannelsPerConvGroup};
  shape.insert(shape.end(), params.kernelShape.begin(),
               params.kernelShape.end());
  DeviceTensor weights(params.inputType, shape,
                       DeviceTensor::Layout::PackedWeights,
                       bufferBytes(plan->plan, MXCONV_BUFFER_WEIGHTS_PACKED));
  weights.packedFor = plan;
  return weights;
}

DeviceTensor createBiases(const DeviceTensor &acts) {
  if (acts.shape().size() < 2)
    throw poputil::poplibs_error("createBiases: activations need at least "
                                 "batch and channel dimensions");
  const std::size_t chans = acts.shape()[1];
  return DeviceTensor(acts.elementType(), {chans},
                      DeviceTensor::Layout::External,
                      chans * acts.elementType().size());
}

DeviceTensor createBiases(const ConvParams &params,
                          const poplar::OptionFlags &options,
                          PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  return DeviceTensor(params.outputType, {params.getNumOutputChans()},
                      DeviceTensor::Layout::External,
                      bufferBytes(plan->plan, MXCONV_BUFFER_BIAS));
}

DeviceTensor createInput(const ConvParams &params,
                         const poplar::OptionFlags &options,
                         PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  return DeviceTensor(params.inputType,
                      actsShape(params.batchSize, params.getNumInputChans(),
                                params.inputFieldShape),
                      DeviceTensor::Layout::ChannelsLast,
                      bufferBytes(plan->plan, MXCONV_BUFFER_INPUT));
}

DeviceTensor createConvOutput(const ConvParams &params,
                              const poplar::OptionFlags &options,
                              PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  return DeviceTensor(params.outputType,
                      actsShape(params.batchSize, params.getNumOutputChans(),
                                params.getOutputFieldShape()),
                      DeviceTensor::Layout::ChannelsLast,
                      bufferBytes(plan->plan, MXCONV_BUFFER_OUTPUT));
}

namespace {

/// verifyInputShapesAndTypes (lib/poplin/Convolution.cpp:105-162).
void verify(const ConvParams &params, const DeviceTensor &in,
            const DeviceTensor &weights, const DeviceTensor *out) {
  const auto expectIn = actsShape(params.batchSize, params.getNumInputChans(),
                                  params.inputFieldShape);
  if (in.shape() != expectIn)
    throw poputil::poplibs_error(
        "Input tensor shape does not match the convolution parameters");
  std::vector<std::size_t> expectW{params.numConvGroups,
                                   params.outputChannelsPerConvGroup,
                                   params.inputChannelsPerConvGroup};
  expectW.insert(expectW.end(), params.kernelShape.begin(),
                 params.kernelShape.end());
  if (weights.shape() != expectW)
    throw poputil::poplibs_error(
        "Weights tensor shape does not match the convolution parameters");
  if (in.elementType() != params.inputType ||
      weights.elementType() != params.inputType)
    throw poputil::poplibs_error("Input and weights element types must equal "
                                 "the parameters' input type");
  if (out) {
    if (out->shape() != actsShape(params.batchSize, params.getNumOutputChans(),
                                  params.getOutputFieldShape()))
      throw poputil::poplibs_error(
          "Output tensor shape does not match the convolution parameters");
    if (out->elementType() != params.outputType)
      throw poputil::poplibs_error(
          "Output element type must equal the parameters' output type");
  }
}

void run(const PlanHandle &plan, const ConvParams &params,
         const DeviceTensor &in, const DeviceTensor &weights,
         const DeviceTensor &out, Stream &prog) {
  // Bring operands into the device layouts if the caller holds them in the
  // external ones (PopLibs rearranges unsuitably laid-out operands the same
  // way, lib/poplin/Convolution.cpp:2569-2628).
  DeviceTensor inCl = in, wPacked = weights, outCl = out;
  if (in.layout() == DeviceTensor::Layout::External) {
    inCl = DeviceTensor(in.elementType(), in.shape(),
                        DeviceTensor::Layout::ChannelsLast, in.bytes());
    check(mxconv_acts_to_internal(plan.plan, in.data(), inCl.data(),
                                  streamOf(prog)));
  }
  if (weights.layout() == DeviceTensor::Layout::PackedWeights)
    requirePackedFor(plan.plan, weights, "weights");
  if (weights.layout() == DeviceTensor::Layout::External) {
    wPacked = DeviceTensor(weights.elementType(), weights.shape(),
                           DeviceTensor::Layout::PackedWeights,
                           bufferBytes(plan.plan, MXCONV_BUFFER_WEIGHTS_PACKED));
    check(mxconv_pack_weights(plan.plan, weights.data(), wPacked.data(),
                              streamOf(prog)));
  }
  if (out.layout() == DeviceTensor::Layout::External)
    outCl = DeviceTensor(out.elementType(), out.shape(),
                         DeviceTensor::Layout::ChannelsLast, out.bytes());
  const std::size_t wsBytes = bufferBytes(plan.plan, MXCONV_BUFFER_WORKSPACE);
  DeviceTensor workspace;
  if (wsBytes)
    workspace = DeviceTensor(poplar::FLOAT, {wsBytes / 4},
                             DeviceTensor::Layout::External, wsBytes);
  if (params.inputType == poplar::QUARTER)
    check(mxconv_fwd_quarter(plan.plan, inCl.data(), in.metadata.byte(),
                             wPacked.data(), weights.metadata.byte(), nullptr,
                             outCl.data(), workspace.data(), wsBytes,
                             streamOf(prog)));
  else
    check(mxconv_fwd(plan.plan, inCl.data(), wPacked.data(), nullptr,
                     outCl.data(), workspace.data(), wsBytes, streamOf(prog)));
  if (out.layout() == DeviceTensor::Layout::External)
    check(mxconv_acts_to_external(plan.plan, outCl.data(), out.data(),
                                  streamOf(prog)));
  // Temporaries are released when this function returns; work already
  // enqueued on the stream must have finished with them by then.
  if (inCl.data() != in.data() || wPacked.data() != weights.data() ||
      outCl.data() != out.data() || wsBytes)
    prog.synchronize();
}

} // namespace

void convolutionWithOutput(const DeviceTensor &in, const DeviceTensor &weights,
                           const DeviceTensor &out, const ConvParams &params,
                           bool transposeAndFlipWeights, Stream &prog,
                           const poplar::OptionFlags &options,
                           PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  if (!transposeAndFlipWeights) {
    verify(params, in, weights, &out);
    run(*plan, params, in, weights, out, prog);
    return;
  }
  // Backward pass: `weights` are the forward pass's,
  // [G][params.inChans][params.outChans][kernel...]; transpose the channel
  // axes and flip the spatial ones first (lib/poplin/Convolution.cpp:
  // 3077-3086).
  if (weights.layout() != DeviceTensor::Layout::External)
    throw poputil::poplibs_error(
        "transposeAndFlipWeights needs the weights in the external layout "
        "(packed weights belong to the plan they were packed for)");
  std::vector<std::size_t> fwdShape{params.numConvGroups,
                                    params.inputChannelsPerConvGroup,
                                    params.outputChannelsPerConvGroup};
  fwdShape.insert(fwdShape.end(), params.kernelShape.begin(),
                  params.kernelShape.end());
  if (weights.shape() != fwdShape)
    throw poputil::poplibs_error(
        "Weights tensor shape does not match the convolution parameters "
        "(expected the forward pass's [G][outChans][inChans][kernel...])");
  std::vector<std::size_t> bwdShape = fwdShape;
  std::swap(bwdShape[1], bwdShape[2]);
  DeviceTensor flipped(weights.elementType(), bwdShape,
                       DeviceTensor::Layout::External, weights.bytes());
  flipped.metadata = weights.metadata;
  weightsTransposeChansFlipXY(weights, flipped, prog);
  verify(params, in, flipped, &out);
  run(*plan, params, in, flipped, out, prog);
  prog.synchronize(); // `flipped` is released on return
}

void weightsTransposeChansFlipXY(const DeviceTensor &weightsIn,
                                 const DeviceTensor &weightsOut, Stream &prog) {
  const auto &si = weightsIn.shape(), &so = weightsOut.shape();
  if (si.size() < 3 || si.size() - 3 > MXCONV_MAX_FIELD_DIMS ||
      so.size() != si.size() || so[0] != si[0] || so[1] != si[2] ||
      so[2] != si[1] ||
      !std::equal(si.begin() + 3, si.end(), so.begin() + 3))
    throw poputil::poplibs_error(
        "weightsTransposeChansFlipXY: weightsOut must be "
        "[G][inChans][outChans][kernel...] for weightsIn "
        "[G][outChans][inChans][kernel...]");
  if (weightsIn.layout() != DeviceTensor::Layout::External ||
      weightsOut.layout() != DeviceTensor::Layout::External ||
      weightsIn.elementType() != weightsOut.elementType())
    throw poputil::poplibs_error(
        "weightsTransposeChansFlipXY: both tensors must be in the external "
        "layout and share an element type");
  // Forward parameters carrying just what the transposition needs.
  ConvParams fwd(weightsIn.elementType(), 1,
                 std::vector<std::size_t>(si.begin() + 3, si.end()),
                 std::vector<std::size_t>(si.begin() + 3, si.end()), si[2],
                 si[1], si[0]);
  mxconv_params c;
  fwd.toC(c);
  check(mxconv_weights_transpose_chans_flip_xy(&c, weightsIn.data(),
                                               weightsOut.data(),
                                               streamOf(prog)));
}

DeviceTensor fullyConnectedWeightTranspose(const DeviceTensor &weights,
                                           const ConvParams &params,
                                           Stream &prog,
                                           const poplar::OptionFlags &options,
                                           PlanningCache *cache) {
  if (params.getNumFieldDims() != 1)
    throw poputil::poplibs_error(
        "fullyConnectedWeightTranspose() expects a 1-d convolution");
  const std::vector<std::size_t> fwdShape{
      params.numConvGroups, params.inputChannelsPerConvGroup,
      params.outputChannelsPerConvGroup, params.kernelShape[0]};
  if (weights.layout() != DeviceTensor::Layout::External ||
      weights.shape() != fwdShape || weights.elementType() != params.inputType)
    throw poputil::poplibs_error(
        "fullyConnectedWeightTranspose: expected the forward pass's weights, "
        "[G][params.inChans][params.outChans][k] in the external layout and "
        "the parameters' input type");
  auto plan = getPlan(params, options, cache);
  const std::vector<std::size_t> bwdShape{fwdShape[0], fwdShape[2], fwdShape[1],
                                          fwdShape[3]};
  DeviceTensor swapped(weights.elementType(), bwdShape,
                       DeviceTensor::Layout::External, weights.bytes());
  swapped.metadata = weights.metadata;
  const std::size_t k = fwdShape[3];
  if (k == 1) {
    check(mxconv_transpose_grouped_matrix(
        weights.elementType().id(), fwdShape[0], fwdShape[1], fwdShape[2],
        weights.data(), swapped.data(), streamOf(prog)));
  } else {
    // The channel axes exchanged with the taps flipped, then every
    // (group, channel pair)'s taps flipped back as a kernel of its own.
    DeviceTensor flipped(weights.elementType(), bwdShape,
                         DeviceTensor::Layout::External, weights.bytes());
    weightsTransposeChansFlipXY(weights, flipped, prog);
    ConvParams each(weights.elementType(), 1, {k}, {k}, 1, 1,
                    fwdShape[0] * fwdShape[1] * fwdShape[2]);
    mxconv_params c;
    each.toC(c);
    check(mxconv_weights_transpose_chans_flip_xy(&c, flipped.data(),
                                                 swapped.data(),
                                                 streamOf(prog)));
    prog.synchronize(); // `flipped` is released on leaving this block
  }
  DeviceTensor packed(weights.elementType(), bwdShape,
                      DeviceTensor::Layout::PackedWeights,
                      bufferBytes(plan->plan, MXCONV_BUFFER_WEIGHTS_PACKED));
  packed.metadata = weights.metadata;
  packed.packedFor = plan;
  check(mxconv_pack_weights(plan->plan, swapped.data(), packed.data(),
                            streamOf(prog)));
  prog.synchronize(); // `swapped` is released on return
  return packed;
}

DeviceTensor convolution(const DeviceTensor &in, const DeviceTensor &weights,
                         const ConvParams &params,
                         bool transposeAndFlipWeights, Stream &prog,
                         const poplar::OptionFlags &options,
                         PlanningCache *cache) {
  DeviceTensor out = createConvOutput(params, options, cache);
  convolutionWithOutput(in, weights, out, params, transposeAndFlipWeights, prog,
                        options, cache);
  return out;
}

void addBias(const DeviceTensor &in, const DeviceTensor &biases, Stream &prog) {
  if (in.shape().size() < 2 || biases.shape().size() != 1 ||
      biases.shape()[0] != in.shape()[1])
    throw poputil::poplibs_error(
        "addBias: bias must have one element per activation channel");
  if (in.elementType() != biases.elementType())
    throw poputil::poplibs_error(
        "addBias: bias and activations must share an element type");
  if (in.layout() != DeviceTensor::Layout::ChannelsLast)
    throw poputil::poplibs_error(
        "addBias: activations must be held channels-last (createInput / "
        "createConvOutput / convolution results are)");
  const std::size_t chans = in.shape()[1];
  const std::size_t outer = chans ? in.numElements() / chans : 0;
  check(mxconv_add_bias(in.elementType().id(), in.data(), biases.data(), outer,
                        chans, streamOf(prog)));
}

void reportPlanInfo(std::ostream &out, const ConvParams &params,
                    const poplar::OptionFlags &options, PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  std::size_t needed = 0;
  check(mxconv_plan_describe(plan->plan, nullptr, 0, &needed));
  std::string text(needed, '\0');
  check(mxconv_plan_describe(plan->plan, &text[0], text.size(), &needed));
  text.resize(needed - 1);
  out << text;
}

PlanCosts reportPlanEstimatedCosts(const ConvParams &params,
                                   const poplar::OptionFlags &options,
                                   PlanningCache *cache) {
  auto plan = getPlan(params, options, cache);
  std::uint64_t cycles = 0, memory = 0;
  check(mxconv_plan_estimated_costs(plan->plan, &cycles, &memory));
  return {cycles == MXCONV_COST_UNKNOWN ? PlanCosts::unknown
                                        : std::size_t(cycles),
          std::size_t(memory)};
}

namespace internal {

std::ostream &operator<<(std::ostream &os, DetailedPlanCosts const &c) {
  os << c.parallelSplit << ' ' << c.serialSplit << '\n';
  c.apply([&](const PlanCosts &phase) {
    os << phase.cycles << ' ' << phase.memory << '\n';
  });
  return os;
}

std::istream &operator>>(std::istream &is, DetailedPlanCosts &c) {
  is >> c.parallelSplit >> c.serialSplit;
  c.apply([&](PlanCosts &phase) { is >> phase.cycles >> phase.memory; });
  return is;
}

DetailedPlanCosts
reportDetailedPlanEstimatedCosts(const ConvParams &params,
                                 const poplar::OptionFlags &options,
                                 PlanningCache *cache) {
  auto plan = detail::getPlan(params, options, cache);
  mxconv_detailed_costs raw{};
  detail::check(mxconv_plan_detailed_costs(plan->plan, &raw));
  auto phase = [](const mxconv_phase_cost &p) {
    return PlanCosts{p.cycles == MXCONV_COST_UNKNOWN ? PlanCosts::unknown
                                                     : std::size_t(p.cycles),
                     std::size_t(p.memory_bytes)};
  };
  DetailedPlanCosts c;
  c.parallelSplit = std::size_t(raw.parallel_split);
  c.serialSplit = std::size_t(raw.serial_split);
  c.rearrangement = phase(raw.rearrangement);
  c.compute = phase(raw.compute);
  c.reduction = phase(raw.reduction);
  c.total = phase(raw.total);
  return c;
}

} // namespace internal

void preplanConvolutions(const std::set<ConvPlanParams> &convs,
                         PlanningCache &cache) {
  preplan(convs, {}, cache);
}

void preplanMatMuls(const std::set<MatMulPlanParams> &matmuls,
                    matmul::PlanningCache &cache) {
  preplan({}, matmuls, cache.getImpl());
}

void preplan(const std::set<ConvPlanParams> &convs,
             const std::set<MatMulPlanParams> &matmuls, PlanningCache &cache) {
  if (convs.empty() && matmuls.empty())
    return;
  MatMulToConvOptions matmulOptions;
  const std::set<ConvPlanParams> matmulConvs =
      matMulGetConvPlanParams(matmuls, matmulOptions);

  // Distinct cache keys that the cache does not hold yet.
  using Key = PlanningCache::Impl::Key;
  struct Job {
    Key key;
    const ConvParams *params;
    std::shared_ptr<PlanHandle> plan;
    std::exception_ptr error;
  };
  std::vector<Job> jobs;
  {
    std::set<Key> seen;
    std::lock_guard<std::mutex> lock(cache.impl->mutex);
    for (const auto *set : {&convs, &matmulConvs})
      for (const auto &conv : *set) {
        if (!std::get<2>(conv))
          throw poputil::poplibs_error(
              "preplan: null pointer to the options");
        Key key{std::get<1>(conv).canonicalize(), *std::get<2>(conv)};
        if (cache.impl->plans.count(key) || !seen.insert(key).second)
          continue;
        jobs.push_back(Job{std::move(key), &std::get<1>(conv), nullptr,
                           nullptr});
      }
  }
  // Plans are independent host computations: make them on as many threads
  // as the host offers (each job writes its own slot), then insert them one
  // after the other (lib/poplin/ConvPlan.cpp:1839-1875).
  const std::size_t workers = std::min<std::size_t>(
      jobs.size(), std::max(1u, std::thread::hardware_concurrency()));
  std::atomic<std::size_t> next{0};
  auto work = [&] {
    for (std::size_t i; (i = next.fetch_add(1)) < jobs.size();) {
      try {
        jobs[i].plan = createPlan(*jobs[i].params, jobs[i].key.second);
      } catch (...) {
        jobs[i].error = std::current_exception();
      }
    }
  };
  std::vector<std::thread> threads;
  for (std::size_t t = 1; t < workers; ++t)
    threads.emplace_back(work);
  work();
  for (auto &t : threads)
    t.join();
  for (const Job &job : jobs)
    if (job.error)
      std::rethrow_exception(job.error);
  std::lock_guard<std::mutex> lock(cache.impl->mutex);
  for (Job &job : jobs)
    cache.impl->plans.emplace(std::move(job.key), std::move(job.plan));
}

void convolutionValidateOptions(const poplar::OptionFlags &options) {
  std::vector<const char *> keys, values;
  for (const auto &kv : options) {
    keys.push_back(kv.first.c_str());
    values.push_back(kv.second.c_str());
  }
  check(mxconv_validate_options(keys.data(), values.data(), keys.size()));
}

void writeTensor(const DeviceTensor &t, const void *host, Stream &prog,
                 const ConvParams &params, const poplar::OptionFlags &options,
                 PlanningCache *cache) {
  hipStream_t s = static_cast<hipStream_t>(prog.handle());
  const std::size_t logicalBytes = t.numElements() * t.elementType().size();
  if (t.layout() == DeviceTensor::Layout::External) {
    if (logicalBytes)
      checkHip(hipMemcpyAsync(t.data(), host, logicalBytes,
                              hipMemcpyHostToDevice, s),
               "hipMemcpyAsync");
    prog.synchronize();
    return;
  }
  auto plan = getPlan(params, options, cache);
  DeviceTensor staging(t.elementType(), t.shape(),
                       DeviceTensor::Layout::External, logicalBytes);
  if (logicalBytes)
    checkHip(hipMemcpyAsync(staging.data(), host, logicalBytes,
                            hipMemcpyHostToDevice, s),
             "hipMemcpyAsync");
  if (t.layout() == DeviceTensor::Layout::PackedWeights) {
    check(mxconv_pack_weights(plan->plan, staging.data(), t.data(),
                              streamOf(prog)));
  } else {
    if (t.shape() != actsShape(params.batchSize, params.getNumInputChans(),
                               params.inputFieldShape))
      throw poputil::poplibs_error(
          "writeTensor: only the convolution's input can be written in "
          "channels-last layout");
    check(mxconv_acts_to_internal(plan->plan, staging.data(), t.data(),
                                  streamOf(prog)));
  }
  prog.synchronize(); // staging is released on return
}

void readTensor(const DeviceTensor &t, void *host, Stream &prog,
                const ConvParams &params, const poplar::OptionFlags &options,
                PlanningCache *cache) {
  hipStream_t s = static_cast<hipStream_t>(prog.handle());
  const std::size_t logicalBytes = t.numElements() * t.elementType().size();
  if (t.layout() == DeviceTensor::Layout::External) {
    if (logicalBytes)
      checkHip(hipMemcpyAsync(host, t.data(), logicalBytes,
                              hipMemcpyDeviceToHost, s),
               "hipMemcpyAsync");
    prog.synchronize();
    return;
  }
  if (t.layout() != DeviceTensor::Layout::ChannelsLast ||
      t.shape() != actsShape(params.batchSize, params.getNumOutputChans(),
                             params.getOutputFieldShape()))
    throw poputil::poplibs_error(
        "readTensor: only the convolution's output can be read back from a "
        "device layout");
  auto plan = getPlan(params, options, cache);
  DeviceTensor staging(t.elementType(), t.shape(),
                       DeviceTensor::Layout::External, logicalBytes);
  check(mxconv_acts_to_external(plan->plan, t.data(), staging.data(),
                                streamOf(prog)));
  if (logicalBytes)
    checkHip(hipMemcpyAsync(host, staging.data(), logicalBytes,
                            hipMemcpyDeviceToHost, s),
             "hipMemcpyAsync");
  prog.synchronize();
}

void writeTensor(const DeviceTensor &t, const void *host, Stream &prog) {
  if (t.layout() != DeviceTensor::Layout::External)
    throw poputil::poplibs_error(
        "writeTensor: a tensor in a device layout needs the parameters of "
        "the plan that laid it out");
  writeTensor(t, host, prog, ConvParams{});
}

void readTensor(const DeviceTensor &t, void *host, Stream &prog) {
  if (t.layout() != DeviceTensor::Layout::External)
    throw poputil::poplibs_error(
        "readTensor: a tensor in a device layout needs the parameters of "
        "the plan that laid it out");
  readTensor(t, host, prog, ConvParams{});
}

} // namespace poplin

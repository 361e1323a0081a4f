// The C ABI declared in mxconv.h: argument checking, translation of C++
// exceptions into status codes, and dispatch to the kernel launchers.
#include "mxconv.h"

#include <hip/hip_runtime.h>

#include "../src/ConvOptions.hpp"
#include "../src/MatMulOptions.hpp"
#include "../src/Plan.hpp"
#include "kernels.hpp"
#include "poplar/exceptions.hpp"
#include "poplin/ConvParams.hpp"
#include "poplin/ConvUtil.hpp"
#include "poputil/exceptions.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <new>
#include <fstream>
#include <sstream>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local std::string lastError;

mxconv_status fail(mxconv_status s, const std::string &message) {
  lastError = message;
  return s;
}

/// Runs `body`, mapping the exceptions of the C++ layer to status codes.
template <class F> mxconv_status guarded(F &&body) {
  try {
    lastError.clear();
    return body();
  } catch (const poplar::invalid_option &e) {
    return fail(MXCONV_INVALID_OPTION, e.what());
  } catch (const poplar::graph_memory_allocation_error &e) {
    return fail(MXCONV_OUT_OF_MEMORY, e.what());
  } catch (const poputil::poplibs_error &e) {
    return fail(MXCONV_INVALID_PARAMS, e.what());
  } catch (const std::bad_alloc &) {
    return fail(MXCONV_OUT_OF_MEMORY, "host allocation failed");
  } catch (const std::exception &e) {
    return fail(MXCONV_INVALID_PARAMS, e.what());
  }
}

#define REQUIRE_ARG(p)                                                         \
  if (!(p))                                                                    \
  return fail(MXCONV_NULL_ARGUMENT, "null argument: " #p)

mxconv_status copyOut(const std::string &text, char *buffer, size_t capacity,
                      size_t *needed) {
  if (needed)
    *needed = text.size() + 1;
  if (buffer && capacity) {
    const size_t n = std::min(capacity - 1, text.size());
    std::memcpy(buffer, text.data(), n);
    buffer[n] = '\0';
  }
  if (buffer && capacity < text.size() + 1)
    return fail(MXCONV_BUFFER_TOO_SMALL, "text truncated");
  return MXCONV_OK;
}

std::vector<std::pair<std::string, std::string>>
collectOptions(const char *const *keys, const char *const *values, size_t n) {
  std::vector<std::pair<std::string, std::string>> flags;
  for (size_t i = 0; i != n; ++i) {
    if (!keys || !values || !keys[i] || !values[i])
      throw poplar::invalid_option("null option key or value");
    flags.emplace_back(keys[i], values[i]);
  }
  return flags;
}

mxconv_status hipStatus(hipError_t e, const char *what) {
  if (e == hipSuccess)
    return MXCONV_OK;
  std::string message = std::string(what) + ": " + hipGetErrorString(e);
  return fail(e == hipErrorOutOfMemory ? MXCONV_OUT_OF_MEMORY
                                       : MXCONV_HIP_ERROR,
              message);
}

void checkDim(const poplin::ConvParams &p, uint32_t dim) {
  if (dim >= p.getNumFieldDims())
    throw poputil::poplibs_error("dimension " + std::to_string(dim) +
                                 " out of range");
}

mxk::QuarterInfo quarterInfo(uint8_t inMeta, uint8_t wMeta) {
  auto scaleOf = [](uint8_t m) {
    int s = m & 0x3f;
    return (s & 0x20) ? s - 64 : s;
  };
  mxk::QuarterInfo q;
  q.inFormat = (inMeta >> 7) & 1;
  q.weightFormat = (wMeta >> 7) & 1;
  q.scale = std::ldexp(1.0f, scaleOf(inMeta) + scaleOf(wMeta));
  return q;
}

/// The argument checks of a forward pass; MXCONV_OK also when there is
/// nothing to compute (no output elements).
mxconv_status checkForward(const mxconv_plan *plan, const void *in,
                           const void *w, const void *out,
                           const void *workspace, size_t workspaceBytes) {
  REQUIRE_ARG(plan);
  if (plan->outputElems == 0)
    return MXCONV_OK;
  REQUIRE_ARG(out);
  if (plan->inputElems != 0)
    REQUIRE_ARG(in);
  if (plan->weightElems != 0)
    REQUIRE_ARG(w);
  if (workspaceBytes < plan->workspaceBytes ||
      (plan->workspaceBytes && !workspace))
    return fail(MXCONV_WORKSPACE_TOO_SMALL,
                "workspace of " + std::to_string(plan->workspaceBytes) +
                    " bytes required");
  return MXCONV_OK;
}

mxconv_status forward(const mxconv_plan *plan, const void *in, const void *w,
                      const void *bias, void *out, void *workspace,
                      size_t workspaceBytes, const mxk::QuarterInfo &q,
                      mxconv_stream stream) {
  const mxconv_status checked =
      checkForward(plan, in, w, out, workspace, workspaceBytes);
  if (checked != MXCONV_OK || plan->outputElems == 0)
    return checked;
  const int inType = plan->params.inputType.id();
  const int outType = plan->params.outputType.id();
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  switch (plan->kernel) {
  case mxconv_plan::Kernel::IGEMM: {
    // Phases of a zero-stuffed input that no tap reaches (a 1x1 layer's
    // backward pass at stride 2: three in four) only write zeros (the bias):
    // where they are half of the phases or more, one fill of the whole output
    // does that and the launch leaves them out.
    size_t deadPhases = 0;
    for (const auto &phase : plan->igemmPhases)
      deadPhases += phase.d.noTaps ? 1 : 0;
    const bool fillAll = deadPhases && 2 * deadPhases >= plan->igemmPhases.size();
    if (plan->outputPadded || fillAll) {
      // zeros (the bias) around the convolution's own outputs
      const mxk::IgemmDesc &g = plan->igemm;
      const uint32_t fullD = g.outFullD ? g.outFullD : g.outD;
      const uint32_t fullH = g.outFullH ? g.outFullH : g.outH,
                     fullW = g.outFullW ? g.outFullW : g.outW;
      const uint32_t insideD =
                         fillAll ? 0
                                 : fullD - plan->outputPadLoD -
                                       plan->outputPadHiD,
                     insideH = fillAll ? 0
                                       : fullH - plan->outputPadLoH -
                                             plan->outputPadHiH,
                     insideW = fillAll ? 0
                                       : fullW - plan->outputPadLoW -
                                             plan->outputPadHiW;
      const mxconv_status st = hipStatus(
          mxk::launchFillOutputPadding(
              outType, out, bias, g.batch, fullD, fullH, fullW,
              plan->outputPadLoD, plan->outputPadLoH, plan->outputPadLoW,
              insideD, insideH, insideW,
              uint32_t(plan->params.getNumOutputChans()), s),
          "output padding fill");
      if (st != MXCONV_OK)
        return st;
    }
    if (plan->thinInputOn)
      return hipStatus(mxk::launchThinInput(plan->thinInput, inType, outType,
                                            in, w, bias, out, s),
                       "thin-input convolution launch");
    if (plan->pointwiseOn)
      return hipStatus(mxk::launchPointwise(plan->pointwise, inType, outType,
                                            in, w, bias, out, q, s),
                       "pointwise convolution launch");
    if (plan->paddedInputChans) {
      // the kernel reads whole 16-byte vectors of channels: give it a copy
      // with the channels of every group filled up with zeros
      const mxk::IgemmDesc &g = plan->igemm;
      char *padded = static_cast<char *>(workspace) + plan->paddedInputOffset;
      const mxconv_status st = hipStatus(
          mxk::launchPadChans(
              in, padded, uint64_t(g.batch) * g.inD * g.inH * g.inW, g.groups,
              uint32_t(plan->params.inputChannelsPerConvGroup),
              g.inChansPerGroup, int(plan->params.inputType.size()), s),
          "channel padding launch");
      if (st != MXCONV_OK)
        return st;
      in = padded;
    }
    if (plan->igemm.patch)
      return hipStatus(mxk::launchIgemmPatch(plan->igemm, inType, outType, in,
                                             w, bias, out, q, s),
                       "implicit-GEMM convolution launch (resident patch)");
    if (!plan->igemmPhases.empty()) {
      // one convolution per phase of the zero-stuffed input, in one launch
      mxk::IgemmFusedItem items[mxk::kIgemmMaxFused];
      size_t count = 0;
      const size_t elemBytes = plan->params.inputType.size();
      for (const auto &phase : plan->igemmPhases) {
        if (fillAll && phase.d.noTaps)
          continue;
        items[count++] = {&phase.d,
                          inType,
                          outType,
                          in,
                          static_cast<const char *>(w) +
                              phase.packedOffset * elemBytes,
                          bias,
                          out,
                          q};
      }
      if (count == 0)
        return MXCONV_OK; // (the fill was all there is)
      return hipStatus(mxk::launchIgemmFused(items, count, s),
                       "implicit-GEMM convolution launch (phases)");
    }
    return hipStatus(mxk::launchIgemm(plan->igemm, inType, outType, in, w,
                                      bias, out, workspace, q, s),
                     "implicit-GEMM convolution launch");
  }
  case mxconv_plan::Kernel::DEPTHWISE:
    return hipStatus(mxk::launchDepthwise(plan->depthwise, inType, outType, in,
                                          w, bias, out, q, s),
                     "depthwise convolution launch");
  case mxconv_plan::Kernel::GENERIC:
    break;
  }
  return hipStatus(mxk::launchGeneric(plan->generic, inType, outType, in, w,
                                      bias, out, q, s),
                   "generic convolution launch");
}

} // namespace

extern "C" {

const char *mxconv_last_error(void) { return lastError.c_str(); }

const char *mxconv_status_string(mxconv_status status) {
  switch (status) {
  case MXCONV_OK:
    return "ok";
  case MXCONV_INVALID_PARAMS:
    return "invalid parameters";
  case MXCONV_INVALID_OPTION:
    return "invalid option";
  case MXCONV_UNSUPPORTED:
    return "unsupported";
  case MXCONV_OUT_OF_MEMORY:
    return "out of memory";
  case MXCONV_WORKSPACE_TOO_SMALL:
    return "workspace too small";
  case MXCONV_BUFFER_TOO_SMALL:
    return "buffer too small";
  case MXCONV_HIP_ERROR:
    return "HIP error";
  case MXCONV_NULL_ARGUMENT:
    return "null argument";
  }
  return "unknown status";
}

mxconv_status mxconv_params_init(mxconv_params *p, int32_t input_type,
                                 int32_t output_type, uint64_t batch_size,
                                 uint32_t num_field_dims,
                                 const uint64_t *input_field_shape,
                                 const uint64_t *kernel_shape,
                                 uint64_t input_channels_per_conv_group,
                                 uint64_t output_channels_per_conv_group,
                                 uint64_t num_conv_groups) {
  REQUIRE_ARG(p);
  return guarded([&] {
    if (num_field_dims > MXCONV_MAX_FIELD_DIMS)
      throw poputil::poplibs_error("too many field dimensions");
    if (num_field_dims && (!input_field_shape || !kernel_shape))
      throw poputil::poplibs_error("null shape");
    if (input_type < 0 || input_type > 2 || output_type < 0 || output_type > 2)
      throw poputil::poplibs_error("unknown element type id");
    poplin::ConvParams cp(
        poplar::Type(input_type), poplar::Type(output_type), batch_size,
        std::vector<std::size_t>(input_field_shape,
                                 input_field_shape + num_field_dims),
        std::vector<std::size_t>(kernel_shape, kernel_shape + num_field_dims),
        input_channels_per_conv_group, output_channels_per_conv_group,
        num_conv_groups);
    cp.toC(*p);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_validate(const mxconv_params *p) {
  REQUIRE_ARG(p);
  return guarded([&] {
    poplin::ConvParams::fromC(*p).validate();
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_canonicalize(const mxconv_params *p,
                                         mxconv_params *canonical) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(canonical);
  return guarded([&] {
    poplin::ConvParams::fromC(*p).canonicalize().toC(*canonical);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_get_gradient_params(const mxconv_params *p,
                                         mxconv_params *gradient) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(gradient);
  return guarded([&] {
    poplin::getGradientParams(poplin::ConvParams::fromC(*p)).toC(*gradient);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_get_weight_update_params(const mxconv_params *p,
                                              mxconv_params *weight_update) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(weight_update);
  return guarded([&] {
    poplin::getWeightUpdateParams(poplin::ConvParams::fromC(*p))
        .toC(*weight_update);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_is_zero_convolution(const mxconv_params *p,
                                                int *is_zero) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(is_zero);
  return guarded([&] {
    *is_zero =
        poplin::isZeroConvolution(poplin::ConvParams::fromC(*p).canonicalize());
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_size(const mxconv_params *p, int32_t query,
                                 uint32_t dim, uint64_t *size) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(size);
  return guarded([&] {
    const auto cp = poplin::ConvParams::fromC(*p);
    cp.validate();
    checkDim(cp, dim);
    switch (query) {
    case MXCONV_TRUNCATED_INPUT_SIZE:
      *size = cp.getTruncatedInputSize(dim);
      break;
    case MXCONV_TRUNCATED_KERNEL_SIZE:
      *size = cp.getTruncatedKernelSize(dim);
      break;
    case MXCONV_TRANSFORMED_INPUT_SIZE:
      *size = cp.getTransformedInputSize(dim);
      break;
    case MXCONV_TRANSFORMED_KERNEL_SIZE:
      *size = cp.getTransformedKernelSize(dim);
      break;
    case MXCONV_UNTRANSFORMED_OUTPUT_SIZE:
      *size = cp.getUntransformedOutputSize(dim);
      break;
    case MXCONV_OUTPUT_SIZE:
      *size = cp.getOutputSize(dim);
      break;
    default:
      throw poputil::poplibs_error("unknown size query");
    }
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_compare(const mxconv_params *a,
                                    const mxconv_params *b, int *order) {
  REQUIRE_ARG(a);
  REQUIRE_ARG(b);
  REQUIRE_ARG(order);
  return guarded([&] {
    const auto pa = poplin::ConvParams::fromC(*a);
    const auto pb = poplin::ConvParams::fromC(*b);
    *order = pa < pb ? -1 : (pa == pb ? 0 : 1);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_hash(const mxconv_params *p, uint64_t *hash) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(hash);
  return guarded([&] {
    *hash = std::hash<poplin::ConvParams>()(poplin::ConvParams::fromC(*p));
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_from_json(const char *json, mxconv_params *p) {
  REQUIRE_ARG(json);
  REQUIRE_ARG(p);
  return guarded([&] {
    std::istringstream is(json);
    poplin::ConvParams cp;
    is >> cp;
    cp.toC(*p);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_params_to_string(const mxconv_params *p, char *buffer,
                                      size_t capacity, size_t *needed) {
  REQUIRE_ARG(p);
  return guarded([&] {
    const auto cp = poplin::ConvParams::fromC(*p);
    cp.validate();
    std::ostringstream os;
    os << cp;
    return copyOut(os.str(), buffer, capacity, needed);
  });
}

mxconv_status mxconv_get_input_index(const mxconv_params *p, uint32_t dim,
                                     uint32_t output_index,
                                     uint32_t kernel_index, uint32_t *index) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(index);
  return guarded([&] {
    const auto cp = poplin::ConvParams::fromC(*p);
    cp.validate();
    checkDim(cp, dim);
    if (output_index >= cp.getOutputSize(dim) ||
        kernel_index >= cp.kernelShape[dim])
      throw poputil::poplibs_error("index out of range");
    *index = poplin::getInputIndex(dim, output_index, kernel_index, cp);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_get_kernel_index(const mxconv_params *p, uint32_t dim,
                                      uint32_t output_index,
                                      uint32_t input_index, uint32_t *index) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(index);
  return guarded([&] {
    const auto cp = poplin::ConvParams::fromC(*p);
    cp.validate();
    checkDim(cp, dim);
    if (output_index >= cp.getOutputSize(dim) ||
        input_index >= cp.inputFieldShape[dim])
      throw poputil::poplibs_error("index out of range");
    *index = poplin::getKernelIndex(dim, output_index, input_index, cp);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_get_range(const mxconv_params *p, int32_t query,
                               uint32_t dim, const uint32_t a[2],
                               const uint32_t b[2], uint32_t result[2]) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(a);
  REQUIRE_ARG(b);
  REQUIRE_ARG(result);
  return guarded([&] {
    const auto cp = poplin::ConvParams::fromC(*p);
    cp.validate();
    checkDim(cp, dim);
    const unsigned outSize = unsigned(cp.getOutputSize(dim));
    const unsigned inSize = unsigned(cp.inputFieldShape[dim]);
    const unsigned kSize = unsigned(cp.kernelShape[dim]);
    auto check = [](const uint32_t r[2], unsigned limit, const char *what) {
      if (r[0] > r[1] || r[1] > limit)
        throw poputil::poplibs_error(std::string(what) + " range out of bounds");
    };
    check(a, outSize, "output");
    poplin::Range r;
    switch (query) {
    case MXCONV_OUTPUT_RANGE_FOR_KERNEL_RANGE:
      check(b, kSize, "kernel");
      r = poplin::getOutputRangeForKernelRange(dim, {a[0], a[1]}, {b[0], b[1]},
                                               cp);
      break;
    case MXCONV_OUTPUT_RANGE_FOR_INPUT_RANGE:
      check(b, inSize, "input");
      r = poplin::getOutputRangeForInputRange(dim, {a[0], a[1]}, {b[0], b[1]},
                                              cp);
      break;
    case MXCONV_INPUT_RANGE:
      check(b, kSize, "kernel");
      r = poplin::getInputRange(dim, poplin::Range{a[0], a[1]},
                                poplin::Range{b[0], b[1]}, cp);
      break;
    case MXCONV_KERNEL_RANGE:
      check(b, inSize, "input");
      r = poplin::getKernelRange(dim, poplin::Range{a[0], a[1]},
                                 poplin::Range{b[0], b[1]}, cp);
      break;
    default:
      throw poputil::poplibs_error("unknown range query");
    }
    result[0] = r.first;
    result[1] = r.second;
    return MXCONV_OK;
  });
}

mxconv_status mxconv_get_number_of_macs(const mxconv_params *p,
                                        uint64_t *macs) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(macs);
  return guarded([&] {
    const auto cp = poplin::ConvParams::fromC(*p);
    cp.validate();
    *macs = poplin::getNumberOfMACs(cp);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_get_fwd_flops(const mxconv_params *p, uint64_t *flops) {
  REQUIRE_ARG(flops);
  uint64_t macs = 0;
  const mxconv_status s = mxconv_get_number_of_macs(p, &macs);
  if (s == MXCONV_OK)
    *flops = 2 * macs;
  return s;
}

mxconv_status mxconv_validate_options(const char *const *keys,
                                      const char *const *values,
                                      size_t num_options) {
  return guarded([&] {
    poplin::ConvOptions options(collectOptions(keys, values, num_options));
    (void)options;
    return MXCONV_OK;
  });
}

namespace {
/// The option planConstraintsOutputFilename: the plan just made, dumped as a
/// complete planConstraints document to <name>_FWD|_BWD|_WU.json
/// (lib/poplin/ConvPlan.cpp:1638-1666, 1764).
void writeConstraintsFile(const mxconv_plan &plan,
                          const poplin::ConvOptions &options) {
  const std::string path = poplin::getPlanConstraintsOutputFile(options);
  if (path.empty())
    return;
  std::ofstream os(path);
  os << plan.constraintsJson() << "\n";
  if (!os.good())
    throw poputil::poplibs_error("planConstraintsOutputFilename: cannot write '" +
                                 path + "'");
}
} // namespace

mxconv_status mxconv_plan_create(const mxconv_params *p,
                                 const char *const *option_keys,
                                 const char *const *option_values,
                                 size_t num_options, mxconv_plan **plan) {
  REQUIRE_ARG(p);
  REQUIRE_ARG(plan);
  *plan = nullptr;
  return guarded([&] {
    poplin::ConvOptions options(
        collectOptions(option_keys, option_values, num_options));
    *plan = new mxconv_plan(
        poplin::makePlan(poplin::ConvParams::fromC(*p), options));
    writeConstraintsFile(**plan, options);
    return MXCONV_OK;
  });
}

void mxconv_plan_destroy(mxconv_plan *plan) { delete plan; }

mxconv_status mxconv_plan_describe(const mxconv_plan *plan, char *buffer,
                                   size_t capacity, size_t *needed) {
  REQUIRE_ARG(plan);
  return guarded([&] {
    std::ostringstream os;
    os << plan->params << plan->describe();
    return copyOut(os.str(), buffer, capacity, needed);
  });
}

mxconv_status mxconv_plan_constraints(const mxconv_plan *plan, char *buffer,
                                      size_t capacity, size_t *needed) {
  REQUIRE_ARG(plan);
  return guarded([&] {
    return copyOut(plan->constraintsJson(), buffer, capacity, needed);
  });
}

namespace {
size_t ownTensorsWorkspaceBytes(const mxconv_plan *plan);

/// Workspace the planned launch sequence needs.  (A weight update pass on
/// the layer's own tensors keeps its partial sums and deltas there, not the
/// intermediates of the pass's convolution.)
size_t estimatedWorkspaceBytes(const mxconv_plan *plan) {
  return plan->denseWeightUpdate || plan->depthwiseWeightUpdate ||
                 plan->weightUpdateProduct
             ? ownTensorsWorkspaceBytes(plan)
             : plan->workspaceBytes;
}
} // namespace

mxconv_status mxconv_plan_estimated_costs(const mxconv_plan *plan,
                                          uint64_t *cycles,
                                          uint64_t *memory_bytes) {
  REQUIRE_ARG(plan);
  REQUIRE_ARG(cycles);
  REQUIRE_ARG(memory_bytes);
  lastError.clear();
  const double us = plan->estimatedMicroseconds();
  *cycles = us < 0 ? MXCONV_COST_UNKNOWN
                   : uint64_t(us * mxconv_plan::kEstimateClockMHz + 0.5);
  *memory_bytes = estimatedWorkspaceBytes(plan);
  return MXCONV_OK;
}

mxconv_status mxconv_plan_detailed_costs(const mxconv_plan *plan,
                                         mxconv_detailed_costs *costs) {
  REQUIRE_ARG(plan);
  REQUIRE_ARG(costs);
  lastError.clear();
  const mxconv_plan::DetailedEstimate e = plan->detailedEstimate();
  *costs = mxconv_detailed_costs{};
  costs->parallel_split = e.parallelSplit;
  costs->serial_split = e.serialSplit;
  costs->rearrangement.memory_bytes = e.rearrangementBytes;
  costs->reduction.memory_bytes = e.reductionBytes;
  costs->total.memory_bytes = estimatedWorkspaceBytes(plan);
  if (!e.known) {
    costs->rearrangement.cycles = costs->compute.cycles =
        costs->reduction.cycles = costs->total.cycles = MXCONV_COST_UNKNOWN;
    return MXCONV_OK;
  }
  auto cyclesOf = [](double us) {
    return uint64_t(us * mxconv_plan::kEstimateClockMHz + 0.5);
  };
  // The kernel takes what rounding leaves, so that the phases add up.
  costs->total.cycles = cyclesOf(e.totalUs());
  costs->rearrangement.cycles =
      std::min(cyclesOf(e.rearrangementUs), costs->total.cycles);
  costs->reduction.cycles =
      std::min(cyclesOf(e.reductionUs),
               costs->total.cycles - costs->rearrangement.cycles);
  costs->compute.cycles = costs->total.cycles - costs->rearrangement.cycles -
                          costs->reduction.cycles;
  return MXCONV_OK;
}

mxconv_status mxconv_plan_buffer_bytes(const mxconv_plan *plan, int32_t which,
                                       size_t *bytes) {
  REQUIRE_ARG(plan);
  REQUIRE_ARG(bytes);
  lastError.clear();
  switch (which) {
  case MXCONV_BUFFER_INPUT:
    *bytes = plan->inputBytes();
    return MXCONV_OK;
  case MXCONV_BUFFER_WEIGHTS_PACKED:
    *bytes = plan->weightPackedBytes();
    return MXCONV_OK;
  case MXCONV_BUFFER_OUTPUT:
    *bytes = plan->outputBytes();
    return MXCONV_OK;
  case MXCONV_BUFFER_BIAS:
    *bytes = plan->biasBytes();
    return MXCONV_OK;
  case MXCONV_BUFFER_WORKSPACE:
    *bytes = plan->workspaceBytes;
    return MXCONV_OK;
  case MXCONV_BUFFER_WEIGHTS_EXTERNAL:
    *bytes = plan->weightBytes();
    return MXCONV_OK;
  }
  return fail(MXCONV_INVALID_PARAMS, "unknown buffer id");
}

namespace {
/// Everything the layout of a plan's packed weights depends on.
std::string packingSignature(const mxconv_plan &p) {
  std::ostringstream os;
  os << int(p.kernel) << '/' << p.params.inputType.toString() << '/'
     << p.weightElems << '/' << p.weightPackedElems << "/cg"
     << p.convGroupsPerGroup;
  if (p.kernel == mxconv_plan::Kernel::IGEMM) {
    os << "/pw" << p.pointwiseOn << "/thin" << p.thinInputOn << "/patch"
       << p.igemm.patch << "/co"
       << p.coPadded << "/k" << p.kPadded << "/ci" << p.paddedInputChans
       << "/sel" << p.kernelSelected;
    auto taps = [&](const mxk::IgemmTapSelection &t) {
      os << '[' << t.kW << ',' << t.firstH << ',' << t.stepH << ','
         << t.countH << ',' << t.firstW << ',' << t.stepW << ',' << t.countW
         << ',' << t.kH << ',' << t.firstD << ',' << t.stepD << ','
         << t.countD << ']';
    };
    if (p.kernelSelected)
      taps(p.igemmTaps);
    for (const auto &phase : p.igemmPhases) {
      os << "/ph" << phase.packedOffset << ':' << phase.kPadded;
      taps(phase.taps);
    }
  }
  return os.str();
}
} // namespace

mxconv_status mxconv_plans_pack_alike(const mxconv_plan *plan,
                                      const mxconv_plan *packed_for,
                                      int32_t *same) {
  REQUIRE_ARG(plan);
  REQUIRE_ARG(packed_for);
  REQUIRE_ARG(same);
  lastError.clear();
  *same = packingSignature(*plan) == packingSignature(*packed_for) ? 1 : 0;
  return MXCONV_OK;
}

mxconv_status mxconv_pack_weights(const mxconv_plan *plan,
                                  const void *weights_external,
                                  void *weights_packed, mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (plan->weightPackedElems == 0)
    return MXCONV_OK;
  REQUIRE_ARG(weights_packed);
  const auto &p = plan->params;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int elemBytes = int(p.inputType.size());
  uint64_t taps = 1;
  for (auto k : p.kernelShape)
    taps *= k;
  if (plan->kernel == mxconv_plan::Kernel::IGEMM) {
    if (plan->weightElems != 0)
      REQUIRE_ARG(weights_external);
    // Conv groups run as one: their block-diagonal weights, in external
    // order, are laid out behind the packed weights first and packed from
    // there as the weights of the fused groups.
    uint32_t groups = uint32_t(p.numConvGroups);
    uint32_t co = uint32_t(p.outputChannelsPerConvGroup);
    uint32_t ci = uint32_t(p.inputChannelsPerConvGroup);
    if (plan->convGroupsPerGroup > 1) {
      const uint32_t f = plan->convGroupsPerGroup;
      void *fused = static_cast<char *>(weights_packed) +
                    plan->weightPackedElems * elemBytes;
      const mxconv_status st = hipStatus(
          mxk::launchFuseGroupWeights(weights_external, fused, groups, f, co,
                                      ci, taps, elemBytes, s),
          "weight packing");
      if (st != MXCONV_OK)
        return st;
      weights_external = fused;
      groups /= f, co *= f, ci *= f;
    }
    if (plan->thinInputOn)
      return hipStatus(mxk::launchPackThinInputWeights(
                           plan->thinInput, weights_external, weights_packed, s),
                       "weight packing");
    if (plan->pointwiseOn)
      return hipStatus(mxk::launchPackPointwiseWeights(
                           plan->pointwise, weights_external, weights_packed, s),
                       "weight packing");
    for (const auto &phase : plan->igemmPhases) {
      const mxconv_status st = hipStatus(
          mxk::launchPackIgemmWeights(
              weights_external,
              static_cast<char *>(weights_packed) +
                  phase.packedOffset * elemBytes,
              groups, co, ci, uint32_t(taps),
              uint32_t(plan->coPadded), uint32_t(phase.kPadded), elemBytes, s,
              false, uint32_t(plan->paddedInputChans), &phase.taps),
          "weight packing");
      if (st != MXCONV_OK)
        return st;
    }
    if (!plan->igemmPhases.empty())
      return MXCONV_OK;
    if (plan->igemm.patch)
      return hipStatus(
          mxk::launchPackIgemmPatchWeights(
              plan->igemm, p.inputType.id(), weights_external, weights_packed,
              uint32_t(taps), s, false,
              plan->kernelSelected ? &plan->igemmTaps : nullptr),
          "weight packing");
    return hipStatus(
        mxk::launchPackIgemmWeights(
            weights_external, weights_packed, groups, co, ci, uint32_t(taps),
            uint32_t(plan->coPadded), uint32_t(plan->kPadded), elemBytes, s,
            false, uint32_t(plan->paddedInputChans),
            plan->kernelSelected ? &plan->igemmTaps : nullptr),
        "weight packing");
  }
  REQUIRE_ARG(weights_external);
  // [G][Co][Ci][K] -> [G][K][Ci][Co]; with Co = Ci = 1 this is also the
  // depthwise kernel's [K][C].
  const uint64_t dims[4] = {p.numConvGroups, p.outputChannelsPerConvGroup,
                            p.inputChannelsPerConvGroup, taps};
  if (plan->kernel == mxconv_plan::Kernel::DEPTHWISE) {
    const uint64_t dwDims[4] = {1, 1, p.numConvGroups, taps};
    const int perm[4] = {0, 1, 3, 2};
    return hipStatus(mxk::launchPermute4(weights_external, weights_packed,
                                         dwDims, perm, elemBytes, s),
                     "weight packing");
  }
  const int perm[4] = {0, 3, 2, 1};
  return hipStatus(mxk::launchPermute4(weights_external, weights_packed, dims,
                                       perm, elemBytes, s),
                   "weight packing");
}

static mxconv_status transposeActs(const mxconv_plan *plan, const void *src,
                                   void *dst, bool input, bool toInternal,
                                   mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  const auto &p = plan->params;
  uint64_t field = 1;
  if (input)
    for (auto s : p.inputFieldShape)
      field *= s;
  else
    for (auto s : p.getOutputFieldShape())
      field *= s;
  const uint64_t chans = input ? p.getNumInputChans() : p.getNumOutputChans();
  if (p.batchSize * field * chans == 0)
    return MXCONV_OK;
  REQUIRE_ARG(src);
  REQUIRE_ARG(dst);
  const int elemBytes = int((input ? p.inputType : p.outputType).size());
  const int perm[4] = {0, 1, 3, 2};
  uint64_t dims[4] = {1, p.batchSize, chans, field};
  if (!toInternal)
    std::swap(dims[2], dims[3]);
  return hipStatus(mxk::launchPermute4(src, dst, dims, perm, elemBytes,
                                       reinterpret_cast<hipStream_t>(stream)),
                   "activation layout conversion");
}

mxconv_status mxconv_acts_to_internal(const mxconv_plan *plan,
                                      const void *acts_external,
                                      void *acts_internal,
                                      mxconv_stream stream) {
  return transposeActs(plan, acts_external, acts_internal, true, true, stream);
}

mxconv_status mxconv_acts_to_external(const mxconv_plan *plan,
                                      const void *out_internal,
                                      void *out_external,
                                      mxconv_stream stream) {
  return transposeActs(plan, out_internal, out_external, false, false, stream);
}

mxconv_status mxconv_fwd(const mxconv_plan *plan, const void *in,
                         const void *weights_packed, const void *bias,
                         void *out, void *workspace, size_t workspace_bytes,
                         mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (plan->params.inputType == poplar::QUARTER)
    return fail(MXCONV_INVALID_PARAMS,
                "quarter inputs carry metadata: call mxconv_fwd_quarter");
  return forward(plan, in, weights_packed, bias, out, workspace,
                 workspace_bytes, mxk::QuarterInfo{}, stream);
}

mxconv_status mxconv_fwd_quarter(const mxconv_plan *plan, const void *in,
                                 uint8_t in_metadata,
                                 const void *weights_packed,
                                 uint8_t weights_metadata, const void *bias,
                                 void *out, void *workspace,
                                 size_t workspace_bytes, mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (plan->params.inputType != poplar::QUARTER)
    return fail(MXCONV_INVALID_PARAMS,
                "mxconv_fwd_quarter needs a plan with quarter inputs");
  return forward(plan, in, weights_packed, bias, out, workspace,
                 workspace_bytes, quarterInfo(in_metadata, weights_metadata),
                 stream);
}

// ---- forward pass that allocates nothing ----------------------------------

namespace {

// Scratch memory of the allocation-free entry point: one array per GPU, part
// of the loaded code object, held until the process ends.
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxScratchDevices = 64;
std::mutex scratchMutex;
void *scratchOfDevice[kMaxScratchDevices] = {};

/// The address of `scratch` on the current device (every GPU holds its own
/// copy at its own address; the array's name is no device address in host
/// code), looked up once per device.
mxconv_status staticScratch(void **ptr) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess)
    return hipStatus(e, "hipGetDevice");
  if (device < 0 || device >= kMaxScratchDevices)
    return fail(MXCONV_UNSUPPORTED, "device ordinal beyond " +
                                        std::to_string(kMaxScratchDevices));
  std::lock_guard<std::mutex> lock(scratchMutex);
  if (!scratchOfDevice[device]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return hipStatus(e != hipSuccess ? e : hipErrorInvalidSymbol,
                       "hipGetSymbolAddress(scratch)");
    scratchOfDevice[device] = p;
  }
  *ptr = scratchOfDevice[device];
  return MXCONV_OK;
}

} // namespace

mxconv_status mxconv_fwd_static_scratch(const mxconv_plan *plan,
                                        const void *in,
                                        const void *weights_packed,
                                        const void *bias, void *out,
                                        mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (plan->params.inputType == poplar::QUARTER)
    return fail(MXCONV_INVALID_PARAMS,
                "quarter inputs carry metadata: call mxconv_fwd_quarter");
  if (plan->workspaceBytes > kStaticScratchBytes)
    return fail(MXCONV_WORKSPACE_TOO_SMALL,
                "the plan needs " + std::to_string(plan->workspaceBytes) +
                    " bytes of scratch memory, the built-in buffer holds " +
                    std::to_string(kStaticScratchBytes) +
                    ": call mxconv_fwd with a workspace");
  void *ws = nullptr;
  if (plan->workspaceBytes) {
    // (every byte a launch reads from its scratch memory it has written
    // before: partial sums and padded copies are stored whole, so nothing has
    // to be cleared between calls)
    const mxconv_status st = staticScratch(&ws);
    if (st != MXCONV_OK)
      return st;
  }
  return forward(plan, in, weights_packed, bias, out, ws,
                 plan->workspaceBytes, mxk::QuarterInfo{}, stream);
}

// ---- several convolutions at once -----------------------------------------

mxconv_status mxconv_multi_fwd(size_t n, const mxconv_plan *const *plans,
                               const void *const *in,
                               const uint8_t *in_metadata,
                               const void *const *weights_packed,
                               const uint8_t *weights_metadata,
                               const void *const *bias, void *const *out,
                               void *const *workspaces,
                               const size_t *workspace_bytes, int parallel,
                               mxconv_stream stream) {
  lastError.clear();
  if (n == 0)
    return MXCONV_OK;
  REQUIRE_ARG(plans);
  REQUIRE_ARG(in);
  REQUIRE_ARG(weights_packed);
  REQUIRE_ARG(out);
  auto quarter = [&](size_t i) {
    return plans[i]->params.inputType == poplar::QUARTER
               ? quarterInfo(in_metadata ? in_metadata[i] : 0,
                             weights_metadata ? weights_metadata[i] : 0)
               : mxk::QuarterInfo{};
  };
  auto workspace = [&](size_t i) {
    return workspaces ? workspaces[i] : nullptr;
  };
  auto workspaceSize = [&](size_t i) {
    return workspace_bytes ? workspace_bytes[i] : size_t(0);
  };
  // Everything is checked before anything is launched.
  for (size_t i = 0; i != n; ++i) {
    const mxconv_status st =
        checkForward(plans[i], in[i], weights_packed[i], out[i], workspace(i),
                     workspaceSize(i));
    if (st != MXCONV_OK)
      return st;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // A convolution can share a launch when the matrix-core kernel runs it.
  // A plan that cuts K into parts does so because the convolution alone has
  // too few tiles for the chip; in company that may no longer hold, so the
  // shared launch runs it with K in one piece (descriptor copies below) when
  // that is estimated to be faster than the members one by one as planned
  // (measured: about 6 us per launch, 0.3 us per k-step of a workgroup, 5 us
  // for the sum of a split K's parts).
  mxk::IgemmDesc unsplit[mxk::kIgemmMaxFused];
  auto tilesOf = [](const mxk::IgemmDesc &d) {
    const uint64_t m = uint64_t(d.batch) * d.outD * d.outH * d.outW;
    return (m + d.blockM - 1) / d.blockM *
           ((d.outChansPerGroup + d.blockN - 1) / d.blockN) * d.groups;
  };
  auto kStepsOf = [](const mxk::IgemmDesc &d) {
    const uint64_t k = uint64_t(d.kD) * d.kH * d.kW * d.inChansPerGroup;
    return (k + d.blockK - 1) / d.blockK;
  };
  auto fusedItem = [&](size_t i, size_t slot, mxk::IgemmFusedItem &item) {
    const mxconv_plan *p = plans[i];
    // (a plan with more to a launch than its one kernel - a padded copy of
    // the input, several phases, an output border to fill - runs on its own)
    if (p->outputElems == 0 || p->kernel != mxconv_plan::Kernel::IGEMM ||
        p->pointwiseOn || p->thinInputOn || p->paddedInputChans ||
        !p->igemmPhases.empty() ||
        p->outputPadded || p->igemm.patch)
      return false;
    unsplit[slot] = p->igemm;
    unsplit[slot].splitK = 1;
    item = {&unsplit[slot],
            p->params.inputType.id(),
            p->params.outputType.id(),
            in[i],
            weights_packed[i],
            bias ? bias[i] : nullptr,
            out[i],
            quarter(i)};
    return true;
  };
  std::vector<bool> done(n, false);
  for (size_t i = 0; i != n; ++i) {
    if (done[i])
      continue;
    done[i] = true;
    mxk::IgemmFusedItem group[mxk::kIgemmMaxFused];
    size_t member[mxk::kIgemmMaxFused] = {i};
    size_t members = 0;
    double alone = 0, together = 0;
    if (parallel && fusedItem(i, 0, group[0])) {
      members = 1;
      for (size_t j = i + 1; j != n && members != mxk::kIgemmMaxFused; ++j) {
        mxk::IgemmFusedItem item;
        if (!done[j] && fusedItem(j, members, item) &&
            mxk::igemmFusable(group[0], item)) {
          member[members] = j;
          group[members++] = item;
        }
      }
      uint64_t tiles = 0, longest = 0;
      for (size_t k = 0; k != members; ++k) {
        const mxk::IgemmDesc &planned = plans[member[k]]->igemm;
        const uint64_t steps = kStepsOf(planned), own = tilesOf(planned);
        const uint64_t rounds = (own * planned.splitK + 255) / 256;
        alone += 6 + 0.3 * double((steps + planned.splitK - 1) /
                                  planned.splitK * rounds) +
                 (planned.splitK != 1 ? 5 : 0);
        tiles += own;
        longest = std::max(longest, steps);
      }
      together = 6 + 0.3 * double(longest * ((tiles + 255) / 256));
    }
    mxconv_status st;
    if (members >= 2 && together < alone) {
      for (size_t k = 0; k != members; ++k)
        done[member[k]] = true;
      st = hipStatus(mxk::launchIgemmFused(group, members, s),
                     "fused implicit-GEMM convolution launch");
    } else {
      st = forward(plans[i], in[i], weights_packed[i],
                   bias ? bias[i] : nullptr, out[i], workspace(i),
                   workspaceSize(i), quarter(i), stream);
    }
    if (st != MXCONV_OK)
      return st;
  }
  return MXCONV_OK;
}

mxconv_status mxconv_multiconv_validate_options(const char *const *keys,
                                                const char *const *values,
                                                size_t num_options,
                                                int *parallel) {
  return guarded([&] {
    int isParallel = 1;
    for (const auto &kv : collectOptions(keys, values, num_options)) {
      const std::string &key = kv.first, &value = kv.second;
      char *end = nullptr;
      if (key == "planType") {
        if (value != "parallel" && value != "serial")
          throw poplar::invalid_option("Invalid value '" + value +
                                       "' for option 'planType': must be "
                                       "parallel or serial");
        isParallel = value == "parallel";
      } else if (key == "perConvReservedTiles") {
        const long v = std::strtol(value.c_str(), &end, 10);
        if (value.empty() || *end != '\0' || v < 0)
          throw poplar::invalid_option(
              "Invalid value '" + value +
              "' for option 'perConvReservedTiles': must be a non-negative "
              "integer");
      } else if (key == "cycleBackOff") {
        (void)std::strtod(value.c_str(), &end);
        if (value.empty() || *end != '\0')
          throw poplar::invalid_option("Invalid value '" + value +
                                       "' for option 'cycleBackOff': must be "
                                       "a number");
      } else {
        throw poplar::invalid_option("Unrecognised option '" + key + "'");
      }
    }
    if (parallel)
      *parallel = isParallel;
    return MXCONV_OK;
  });
}

// ---- matrix multiplication -------------------------------------------------

} // extern "C"

namespace {

poplin::ConvParams matMulParams(int32_t inputType, int32_t outputType,
                                uint64_t groups, uint64_t m, uint64_t k,
                                uint64_t n) {
  mxconv_params c{};
  c.input_type = inputType;
  c.output_type = outputType;
  const poplin::ConvParams types = poplin::ConvParams::fromC(c); // checks ids
  return poplin::ConvParams(types.inputType, types.outputType, m, {1}, {1}, k,
                            n, groups);
}

/// True when `plan` has the shape mxconv_matmul_params produces.
bool isMatMulPlan(const mxconv_plan *plan) {
  const auto &p = plan->params;
  for (auto s : p.inputFieldShape)
    if (s != 1)
      return false;
  for (auto s : p.kernelShape)
    if (s != 1)
      return false;
  return p == poplin::ConvParams(p.inputType, p.outputType, p.batchSize,
                                 p.inputFieldShape, p.kernelShape,
                                 p.inputChannelsPerConvGroup,
                                 p.outputChannelsPerConvGroup, p.numConvGroups);
}

} // namespace

extern "C" {

mxconv_status mxconv_matmul_params(int32_t input_type, int32_t output_type,
                                   uint64_t groups, uint64_t m, uint64_t k,
                                   uint64_t n, mxconv_params *p) {
  REQUIRE_ARG(p);
  return guarded([&] {
    matMulParams(input_type, output_type, groups, m, k, n).toC(*p);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_matmul_validate_options(const char *const *keys,
                                             const char *const *values,
                                             size_t num_options) {
  return guarded([&] {
    poplin::ConvOptions options(poplin::matMulToConvOptions(
        collectOptions(keys, values, num_options)));
    (void)options;
    return MXCONV_OK;
  });
}

mxconv_status mxconv_matmul_plan_create(int32_t input_type, int32_t output_type,
                                        uint64_t groups, uint64_t m, uint64_t k,
                                        uint64_t n,
                                        const char *const *option_keys,
                                        const char *const *option_values,
                                        size_t num_options, mxconv_plan **plan) {
  REQUIRE_ARG(plan);
  *plan = nullptr;
  return guarded([&] {
    poplin::ConvOptions options(poplin::matMulToConvOptions(
        collectOptions(option_keys, option_values, num_options)));
    *plan = new mxconv_plan(poplin::makePlan(
        matMulParams(input_type, output_type, groups, m, k, n), options));
    return MXCONV_OK;
  });
}

mxconv_status mxconv_matmul_pack_rhs(const mxconv_plan *plan, const void *rhs,
                                     void *weights_packed,
                                     mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (!isMatMulPlan(plan))
    return fail(MXCONV_INVALID_PARAMS,
                "not a matrix-multiplication plan (field and kernel {1}, "
                "identity transforms)");
  if (plan->weightPackedElems == 0)
    return MXCONV_OK;
  REQUIRE_ARG(weights_packed);
  if (plan->weightElems != 0)
    REQUIRE_ARG(rhs);
  const auto &p = plan->params;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int elemBytes = int(p.inputType.size());
  if (plan->kernel == mxconv_plan::Kernel::IGEMM) {
    if (plan->pointwiseOn)
      return hipStatus(mxk::launchPackPointwiseWeights(plan->pointwise, rhs,
                                                       weights_packed, s, true),
                       "weight packing");
    if (plan->igemm.patch)
      return hipStatus(mxk::launchPackIgemmPatchWeights(
                           plan->igemm, p.inputType.id(), rhs, weights_packed,
                           1, s, true),
                       "weight packing");
    return hipStatus(
        mxk::launchPackIgemmWeights(
            rhs, weights_packed, uint32_t(p.numConvGroups),
            uint32_t(p.outputChannelsPerConvGroup),
            uint32_t(p.inputChannelsPerConvGroup), 1, uint32_t(plan->coPadded),
            uint32_t(plan->kPadded), elemBytes, s, true,
            uint32_t(plan->paddedInputChans)),
        "weight packing");
  }
  // Generic kernel: packed = [G][1][Ci][Co], which is B itself.  Depthwise
  // kernel (k = n = 1): packed = [1][G], again B itself.
  return hipStatus(hipMemcpyAsync(weights_packed, rhs, plan->weightBytes(),
                                  hipMemcpyDeviceToDevice, s),
                   "weight packing");
}

} // extern "C"

namespace {

mxconv_status shuffleGroups(const mxconv_plan *plan, const void *src, void *dst,
                            bool toInternal, mxconv_stream stream) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (!isMatMulPlan(plan))
    return fail(MXCONV_INVALID_PARAMS,
                "not a matrix-multiplication plan (field and kernel {1}, "
                "identity transforms)");
  const auto &p = plan->params;
  const uint64_t g = p.numConvGroups, m = p.batchSize;
  const uint64_t c = toInternal ? p.inputChannelsPerConvGroup
                                : p.outputChannelsPerConvGroup;
  if (g * m * c == 0)
    return MXCONV_OK;
  REQUIRE_ARG(src);
  REQUIRE_ARG(dst);
  const int elemBytes =
      int(toInternal ? p.inputType.size() : p.outputType.size());
  // [G][M][C] -> [M][G][C] or back: swap the two leading axes.
  const uint64_t dims[4] = {1, toInternal ? g : m, toInternal ? m : g, c};
  const int perm[4] = {0, 2, 1, 3};
  return hipStatus(mxk::launchPermute4(src, dst, dims, perm, elemBytes,
                                       reinterpret_cast<hipStream_t>(stream)),
                   "matrix group shuffle");
}

} // namespace

extern "C" {

mxconv_status mxconv_matmul_lhs_to_internal(const mxconv_plan *plan,
                                            const void *lhs, void *acts_internal,
                                            mxconv_stream stream) {
  return shuffleGroups(plan, lhs, acts_internal, true, stream);
}

mxconv_status mxconv_matmul_out_to_external(const mxconv_plan *plan,
                                            const void *out_internal,
                                            void *result, mxconv_stream stream) {
  return shuffleGroups(plan, out_internal, result, false, stream);
}

mxconv_status mxconv_weights_transpose_chans_flip_xy(const mxconv_params *p,
                                                     const void *weights_in,
                                                     void *weights_out,
                                                     mxconv_stream stream) {
  REQUIRE_ARG(p);
  lastError.clear();
  poplin::ConvParams params;
  const mxconv_status st = guarded([&] {
    params = poplin::ConvParams::fromC(*p);
    params.validate();
    return MXCONV_OK;
  });
  if (st != MXCONV_OK)
    return st;
  uint64_t elems = params.numConvGroups * params.outputChannelsPerConvGroup *
                   params.inputChannelsPerConvGroup;
  uint32_t shape[MXCONV_MAX_FIELD_DIMS] = {};
  for (std::size_t d = 0; d != params.kernelShape.size(); ++d) {
    shape[d] = uint32_t(params.kernelShape[d]);
    elems *= params.kernelShape[d];
  }
  if (elems == 0)
    return MXCONV_OK;
  REQUIRE_ARG(weights_in);
  REQUIRE_ARG(weights_out);
  return hipStatus(
      mxk::launchWeightsTransposeChansFlipXY(
          weights_in, weights_out, params.numConvGroups,
          params.outputChannelsPerConvGroup, params.inputChannelsPerConvGroup,
          uint32_t(params.kernelShape.size()), shape,
          int(params.inputType.size()), reinterpret_cast<hipStream_t>(stream)),
      "weight transposition");
}

mxconv_status mxconv_transpose_grouped_matrix(int32_t type, uint64_t groups,
                                              uint64_t rows, uint64_t cols,
                                              const void *src, void *dst,
                                              mxconv_stream stream) {
  lastError.clear();
  if (type != MXCONV_QUARTER && type != MXCONV_HALF && type != MXCONV_FLOAT)
    return fail(MXCONV_INVALID_PARAMS, "unknown element type");
  if (groups * rows * cols == 0)
    return MXCONV_OK;
  REQUIRE_ARG(src);
  REQUIRE_ARG(dst);
  const uint64_t dims[4] = {1, groups, rows, cols};
  const int perm[4] = {0, 1, 3, 2};
  const int elemBytes = type == MXCONV_FLOAT ? 4 : type == MXCONV_HALF ? 2 : 1;
  return hipStatus(mxk::launchPermute4(src, dst, dims, perm, elemBytes,
                                       reinterpret_cast<hipStream_t>(stream)),
                   "matrix transposition");
}

mxconv_status mxconv_scaled_add_to(int32_t type, void *c, float scale_c,
                                   const void *product, float scale_product,
                                   uint64_t elems, mxconv_stream stream) {
  lastError.clear();
  if (type != MXCONV_HALF && type != MXCONV_FLOAT)
    return fail(MXCONV_INVALID_PARAMS,
                "scaled add takes half or float tensors");
  if (elems == 0)
    return MXCONV_OK;
  REQUIRE_ARG(c);
  REQUIRE_ARG(product);
  return hipStatus(mxk::launchScaledAdd(type, c, scale_c, product,
                                        scale_product, elems,
                                        reinterpret_cast<hipStream_t>(stream)),
                   "scaled add");
}

mxconv_status mxconv_add_bias(int32_t type, void *acts_internal,
                              const void *bias, uint64_t outer_elems,
                              uint64_t channels, mxconv_stream stream) {
  lastError.clear();
  if (outer_elems * channels == 0)
    return MXCONV_OK;
  REQUIRE_ARG(acts_internal);
  REQUIRE_ARG(bias);
  if (type != MXCONV_HALF && type != MXCONV_FLOAT)
    return fail(MXCONV_INVALID_PARAMS, "bias add takes half or float tensors");
  return hipStatus(mxk::launchAddBias(type, acts_internal, bias, outer_elems,
                                      channels,
                                      reinterpret_cast<hipStream_t>(stream)),
                   "bias add");
}

} // extern "C"

namespace {

size_t alignUp(size_t v) { return (v + 255) & ~size_t(255); }

/// Where the weight update pass keeps its intermediates in the workspace.
struct WuWorkspace {
  size_t input, weightsExternal, weightsPacked, output, deltas, planWorkspace,
      fusedDeltas, total;
};

/// Bytes of the weight deltas the pass hands back (of the layer's own groups,
/// where the plan is for the layer with several groups taken as one).
size_t wuResultBytes(const mxconv_plan *plan) {
  return plan->outputBytes() / plan->wuGroupsPerGroup;
}

WuWorkspace wuWorkspace(const mxconv_plan *plan) {
  WuWorkspace w{};
  size_t at = 0;
  auto take = [&](size_t bytes) {
    const size_t offset = at;
    at += alignUp(bytes);
    return offset;
  };
  // (groups taken as one: the fused layer's deltas, whose diagonal blocks
  // are the result)
  if (plan->wuGroupsPerGroup > 1)
    w.fusedDeltas = take(plan->outputBytes());
  if (plan->depthwiseWeightUpdate) {
    // the depthwise weight-delta kernel reads the layer's tensors as they
    // are: only its partial sums and, for the update, the deltas
    w.planWorkspace =
        take(mxk::depthwiseWeightDeltaWorkspaceBytes(plan->depthwiseForward));
    w.deltas = take(wuResultBytes(plan));
    w.total = at;
    return w;
  }
  if (plan->denseWeightUpdate) {
    w.planWorkspace = take(mxk::wuTapWorkspaceBytes(plan->denseForward));
    w.deltas = take(wuResultBytes(plan));
    w.total = at;
    return w;
  }
  if (const mxconv_plan *product = plan->weightUpdateProduct.get()) {
    // transposed deltas [Co][batch], the activations packed as the
    // product's right-hand side, the product's own workspace
    w.input = take(product->inputBytes());
    w.weightsPacked = take(product->weightPackedBytes());
    w.planWorkspace = take(product->workspaceBytes);
    w.deltas = take(wuResultBytes(plan));
    w.total = at;
    return w;
  }
  w.input = take(plan->inputBytes());
  w.weightsExternal = take(plan->weightBytes());
  w.weightsPacked = take(plan->weightPackedBytes());
  w.output = take(plan->outputBytes());
  w.deltas = take(wuResultBytes(plan));
  w.planWorkspace = take(plan->workspaceBytes);
  w.total = at;
  return w;
}

size_t ownTensorsWorkspaceBytes(const mxconv_plan *plan) {
  return wuWorkspace(plan).total;
}

uint64_t product(const std::vector<std::size_t> &shape) {
  uint64_t n = 1;
  for (auto s : shape)
    n *= s;
  return n;
}

mxconv_status fusedWeightDeltas(const mxconv_plan *plan, const void *zDeltas,
                                const void *acts, void *deltasOut, char *ws,
                                mxconv_stream stream);

/// The pass's result into `deltasOut`, [G][Co][Ci][kernel] of the layer.
mxconv_status weightDeltas(const mxconv_plan *plan, const void *zDeltas,
                           const void *acts, void *deltasOut, char *ws,
                           mxconv_stream stream) {
  const unsigned f = plan->wuGroupsPerGroup;
  if (f == 1)
    return fusedWeightDeltas(plan, zDeltas, acts, deltasOut, ws, stream);
  // Planned for the layer with f groups taken as one: that layer's deltas
  // into the workspace, their diagonal blocks out.
  char *fused = ws + wuWorkspace(plan).fusedDeltas;
  const mxconv_status st =
      fusedWeightDeltas(plan, zDeltas, acts, fused, ws, stream);
  if (st != MXCONV_OK)
    return st;
  const auto &p = plan->params;
  uint64_t taps = 1;
  for (auto k : p.getOutputFieldShape())
    taps *= k;
  return hipStatus(
      mxk::launchUnfuseGroupWeights(
          fused, deltasOut, uint64_t(p.numConvGroups) * f, f,
          p.outputChannelsPerConvGroup / f, p.batchSize / f, taps,
          int(p.outputType.size()), reinterpret_cast<hipStream_t>(stream)),
      "weight deltas of the layer's own groups");
}

/// The weight deltas of the layer the plan was made for.
mxconv_status fusedWeightDeltas(const mxconv_plan *plan, const void *zDeltas,
                                const void *acts, void *deltasOut, char *ws,
                                mxconv_stream stream) {
  // The pass's convolution (lib/poplin/Convolution.cpp:3437-3483): batch =
  // forward input channels, input channels = forward batch, kernel = forward
  // output field, output field = forward kernel.
  const auto &p = plan->params;
  const uint64_t G = p.numConvGroups, Ci = p.batchSize,
                 B = p.inputChannelsPerConvGroup,
                 Co = p.outputChannelsPerConvGroup;
  const uint64_t X = product(p.inputFieldShape), Y = product(p.kernelShape),
                 K = product(p.getOutputFieldShape());
  const int inBytes = int(p.inputType.size());
  const int outBytes = int(p.outputType.size());
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const WuWorkspace w = wuWorkspace(plan);
  if (G * Co * Ci * K == 0)
    return MXCONV_OK;
  if (plan->depthwiseWeightUpdate)
    return hipStatus(mxk::launchDepthwiseWeightDeltas(
                         plan->depthwiseForward, p.outputType.id(), acts,
                         zDeltas, ws + w.planWorkspace, deltasOut, s),
                     "depthwise weight deltas");
  if (plan->denseWeightUpdate)
    return hipStatus(mxk::launchWuTap(plan->denseForward, p.outputType.id(),
                                      acts, zDeltas, ws + w.planWorkspace,
                                      deltasOut, s),
                     "matrix-core weight deltas");
  mxconv_status st;
  if (const mxconv_plan *product = plan->weightUpdateProduct.get()) {
    // No spatial extent: deltas[co][ci] = sum over the batch of
    // dZ[b][co] * x[b][ci] - transpose(dZ) [Co][B] times x [B][Ci], and the
    // result is in weight order as it is.
    st = hipStatus(mxk::launchSwapBatchChans(zDeltas, ws + w.input,
                                             uint32_t(B), 1, 1, uint32_t(Co),
                                             B, B, B, inBytes, s),
                   "delta rearrangement");
    if (st != MXCONV_OK)
      return st;
    st = mxconv_matmul_pack_rhs(product, acts, ws + w.weightsPacked, stream);
    if (st != MXCONV_OK)
      return st;
    return forward(product, ws + w.input, ws + w.weightsPacked, nullptr,
                   deltasOut, ws + w.planWorkspace, product->workspaceBytes,
                   mxk::QuarterInfo{}, stream);
  }
  // activations [B][X][G][Ci] -> the pass's input [Ci][X][G][B]
  const mxk::SwapBatchChans actsSwap{
      acts,        ws + w.input, uint32_t(B), uint32_t(X), uint32_t(G),
      uint32_t(Ci), B,           X * G * B,   G * B};
  const bool direct = plan->kernel == mxconv_plan::Kernel::IGEMM &&
                      !plan->pointwiseOn && !plan->thinInputOn &&
                      !plan->paddedInputChans &&
                      plan->igemmPhases.empty() && !plan->kernelSelected &&
                      !plan->igemm.patch &&
                      // (a padded output field - the forward kernel was
                      // truncated - is filled by the general path)
                      !plan->outputPadded;
  if (direct) {
    // deltas [B][Y][G][Co] -> straight into the matrix-core kernel's packed
    // weights [G][coPadded][kPadded], k = y * B + b; both rearrangements in
    // one launch
    if (plan->coPadded != Co || plan->kPadded != Y * B) {
      st = hipStatus(mxk::launchZero(ws + w.weightsPacked,
                                     alignUp(plan->weightPackedBytes()), s),
                     "delta rearrangement");
      if (st != MXCONV_OK)
        return st;
    }
    const mxk::SwapBatchChans deltasSwap{
        zDeltas,
        ws + w.weightsPacked,
        uint32_t(B),
        uint32_t(Y),
        uint32_t(G),
        uint32_t(Co),
        uint64_t(plan->coPadded) * plan->kPadded,
        plan->kPadded,
        B};
    st = hipStatus(
        mxk::launchSwapBatchChansPair(actsSwap, deltasSwap, inBytes, s),
        "activation and delta rearrangement");
    if (st != MXCONV_OK)
      return st;
    // The pass's output [Ci][K][G][Co] is wanted in weight order
    // [G][Co][Ci][K] - its transpose as a matrix: the kernel (or, with K
    // split, the sum of the parts) writes it that way.
    mxk::IgemmDesc transposed = plan->igemm;
    transposed.outTransposed = 1;
    return hipStatus(
        mxk::launchIgemm(transposed, p.inputType.id(), p.outputType.id(),
                         ws + w.input, ws + w.weightsPacked, nullptr,
                         deltasOut, ws + w.planWorkspace, mxk::QuarterInfo{},
                         s),
        "weight delta convolution launch");
  } else {
    st = hipStatus(mxk::launchSwapBatchChans(
                       actsSwap.src, actsSwap.dst, actsSwap.batch,
                       actsSwap.pixels, actsSwap.groups, actsSwap.chans,
                       actsSwap.strideG, actsSwap.strideC, actsSwap.strideP,
                       inBytes, s),
                   "activation rearrangement");
    if (st != MXCONV_OK)
      return st;
    if (plan->weightElems) {
      // deltas [B][Y][G][Co] -> the pass's weights [G][Co][B][Y]
      const uint64_t dims[4] = {B, Y, G, Co};
      const int perm[4] = {2, 3, 0, 1};
      st = hipStatus(mxk::launchPermute4(zDeltas, ws + w.weightsExternal, dims,
                                         perm, inBytes, s),
                     "delta rearrangement");
      if (st != MXCONV_OK)
        return st;
    }
    st = mxconv_pack_weights(plan, ws + w.weightsExternal,
                             ws + w.weightsPacked, stream);
    if (st != MXCONV_OK)
      return st;
  }
  st = forward(plan, ws + w.input, ws + w.weightsPacked, nullptr,
               ws + w.output, ws + w.planWorkspace, plan->workspaceBytes,
               mxk::QuarterInfo{}, stream);
  if (st != MXCONV_OK)
    return st;
  // the pass's output [Ci][K][G][Co] -> weight order [G][Co][Ci][K]
  const uint64_t dims[4] = {Ci, K, G, Co};
  const int perm[4] = {2, 3, 0, 1};
  return hipStatus(mxk::launchPermute4(ws + w.output, deltasOut, dims, perm,
                                       outBytes, s),
                   "weight delta rearrangement");
}

mxconv_status checkWuCall(const mxconv_plan *plan, const void *zDeltas,
                          const void *acts, const void *result,
                          const void *workspace, size_t workspaceBytes) {
  REQUIRE_ARG(plan);
  lastError.clear();
  if (plan->params.inputType == poplar::QUARTER)
    return fail(MXCONV_UNSUPPORTED,
                "the weight update pass takes half or float tensors");
  if (plan->outputElems == 0)
    return MXCONV_OK;
  REQUIRE_ARG(result);
  if (plan->inputElems)
    REQUIRE_ARG(acts);
  if (plan->weightElems)
    REQUIRE_ARG(zDeltas);
  const size_t need = wuWorkspace(plan).total;
  if (workspaceBytes < need || (need && !workspace))
    return fail(MXCONV_WORKSPACE_TOO_SMALL,
                "workspace of " + std::to_string(need) + " bytes required");
  return MXCONV_OK;
}

} // namespace

extern "C" {

mxconv_status mxconv_weight_update_plan_create(const mxconv_params *fwd,
                                               const char *const *option_keys,
                                               const char *const *option_values,
                                               size_t num_options,
                                               mxconv_plan **plan) {
  REQUIRE_ARG(fwd);
  REQUIRE_ARG(plan);
  *plan = nullptr;
  return guarded([&] {
    poplin::ConvOptions options(
        collectOptions(option_keys, option_values, num_options));
    options = poplin::getWeightUpdateOptions(options);
    *plan = new mxconv_plan(poplin::makePlan(
        poplin::getWeightUpdateParams(poplin::ConvParams::fromC(*fwd)),
        options));
    // A layer without spatial extent (every field and kernel dimension 1,
    // one group): its deltas as one matrix product [Co] x [batch] x [Ci] on
    // the transposed deltas - where nothing in the constraints names a
    // kernel or tile for the pass's own convolution.
    mxconv_plan &made = **plan;
    const auto &pc = options.planConstraints;
    const auto &wp = made.params; // batch = Ci, input channels = the batch
    const bool shapeOk =
        isMatMulPlan(&made) && wp.numConvGroups == 1 && !made.zeroConv &&
        made.outputElems != 0 && made.inputElems != 0 &&
        made.wuGroupsPerGroup == 1 && !made.depthwiseWeightUpdate &&
        wp.inputType != poplar::QUARTER;
    const bool unconstrained =
        pc.weightDeltas == -1 && pc.kernel.empty() &&
        pc.method == poplin::PlanConstraints::Method::ANY && !pc.blockM &&
        !pc.blockN && !pc.blockK && !pc.splitK && !pc.stages &&
        pc.patch < 0 && pc.pointwise < 0;
    if (pc.weightDeltas == 2 && !shapeOk)
      throw poplar::invalid_option(
          "planConstraints gfx950 weightDeltas 2: the deltas are one matrix "
          "product only for a layer without spatial extent (every field and "
          "kernel dimension 1, nothing padded or strided) and one group, of "
          "half or float tensors");
    if (shapeOk && (pc.weightDeltas == 2 || unconstrained)) {
      poplin::ConvOptions productOptions = options;
      productOptions.pass = poplin::Pass::NONE_MATMUL;
      productOptions.planConstraints = poplin::PlanConstraints{};
      made.weightUpdateProduct = std::make_shared<const mxconv_plan>(
          poplin::makePlan(
              matMulParams(wp.inputType.id(), wp.outputType.id(), 1,
                           wp.outputChannelsPerConvGroup,
                           wp.inputChannelsPerConvGroup, wp.batchSize),
              productOptions));
      made.denseWeightUpdate = false;
    }
    writeConstraintsFile(**plan, options);
    return MXCONV_OK;
  });
}

mxconv_status mxconv_weight_update_workspace_bytes(const mxconv_plan *plan,
                                                   size_t *bytes) {
  REQUIRE_ARG(plan);
  REQUIRE_ARG(bytes);
  lastError.clear();
  *bytes = wuWorkspace(plan).total;
  return MXCONV_OK;
}

mxconv_status mxconv_calculate_weight_deltas(const mxconv_plan *plan,
                                             const void *z_deltas_internal,
                                             const void *acts_internal,
                                             void *weight_deltas_external,
                                             void *workspace,
                                             size_t workspace_bytes,
                                             mxconv_stream stream) {
  const mxconv_status st =
      checkWuCall(plan, z_deltas_internal, acts_internal,
                  weight_deltas_external, workspace, workspace_bytes);
  if (st != MXCONV_OK || plan->outputElems == 0)
    return st;
  return weightDeltas(plan, z_deltas_internal, acts_internal,
                      weight_deltas_external, static_cast<char *>(workspace),
                      stream);
}

mxconv_status mxconv_convolution_weight_update(const mxconv_plan *plan,
                                               const void *z_deltas_internal,
                                               void *weights_external,
                                               const void *acts_internal,
                                               float scale, void *workspace,
                                               size_t workspace_bytes,
                                               mxconv_stream stream) {
  mxconv_status st = checkWuCall(plan, z_deltas_internal, acts_internal,
                                 weights_external, workspace, workspace_bytes);
  if (st != MXCONV_OK || plan->outputElems == 0)
    return st;
  if (plan->params.outputType != plan->params.inputType)
    return fail(MXCONV_INVALID_PARAMS,
                "the weight update needs a plan whose output type is the "
                "weights' type");
  char *ws = static_cast<char *>(workspace);
  char *deltas = ws + wuWorkspace(plan).deltas;
  st = weightDeltas(plan, z_deltas_internal, acts_internal, deltas, ws, stream);
  if (st != MXCONV_OK)
    return st;
  return hipStatus(mxk::launchScaledAdd(plan->params.outputType.id(),
                                        weights_external, 1.f, deltas, scale,
                                        plan->outputElems /
                                            plan->wuGroupsPerGroup,
                                        reinterpret_cast<hipStream_t>(stream)),
                   "weight update");
}

mxconv_status mxconv_bias_update_workspace_bytes(uint64_t outer_elems,
                                                 uint64_t channels,
                                                 size_t *bytes) {
  REQUIRE_ARG(bytes);
  lastError.clear();
  *bytes = mxk::biasUpdateWorkspaceBytes(outer_elems, channels);
  return MXCONV_OK;
}

mxconv_status mxconv_convolution_bias_update(int32_t deltas_type,
                                             const void *z_deltas_internal,
                                             uint64_t outer_elems,
                                             uint64_t channels,
                                             int32_t bias_type, void *biases,
                                             float scale, void *workspace,
                                             size_t workspace_bytes,
                                             mxconv_stream stream) {
  lastError.clear();
  for (int32_t t : {deltas_type, bias_type})
    if (t != MXCONV_HALF && t != MXCONV_FLOAT)
      return fail(MXCONV_INVALID_PARAMS,
                  "the bias update takes half or float tensors");
  if (channels == 0)
    return MXCONV_OK;
  REQUIRE_ARG(biases);
  if (outer_elems)
    REQUIRE_ARG(z_deltas_internal);
  const size_t need = mxk::biasUpdateWorkspaceBytes(outer_elems, channels);
  if (workspace_bytes < need || (need && !workspace))
    return fail(MXCONV_WORKSPACE_TOO_SMALL,
                "workspace of " + std::to_string(need) + " bytes required");
  return hipStatus(mxk::launchBiasUpdate(deltas_type, z_deltas_internal,
                                         outer_elems, channels, bias_type,
                                         biases, scale, workspace,
                                         reinterpret_cast<hipStream_t>(stream)),
                   "bias update");
}

} // extern "C"

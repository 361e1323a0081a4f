// Helpers shared by the translation units of the C++ poplin layer: C ABI
// status -> exception, plan handles and the planning cache lookup.
#ifndef poplibs_amd_LayerInternal_hpp
#define poplibs_amd_LayerInternal_hpp
#include "mxconv.h"
#include "poplin/Convolution.hpp"

#include <memory>

namespace poplin {
namespace detail {

/// Throws what the reference would for a failing C ABI call
/// (poputil::poplibs_error, poplar::invalid_option,
/// poplar::graph_memory_allocation_error).
void check(mxconv_status s);

struct PlanHandle {
  mxconv_plan *plan = nullptr;
  explicit PlanHandle(mxconv_plan *p) : plan(p) {}
  ~PlanHandle() { mxconv_plan_destroy(plan); }
  PlanHandle(const PlanHandle &) = delete;
  PlanHandle &operator=(const PlanHandle &) = delete;
};

/// The plan for (params, options), from `cache` when given.
std::shared_ptr<PlanHandle> getPlan(const ConvParams &params,
                                    const poplar::OptionFlags &options,
                                    PlanningCache *cache);
std::size_t bufferBytes(const mxconv_plan *plan, mxconv_buffer which);
/// Throws unless `packed` (a PackedWeights tensor) was arranged for a plan
/// that packs as `plan` does - same kernel, tiling, padding, operand order.
/// A buffer of the right size arranged for another kernel would be read in
/// the wrong operand order.  (PopLibs would rearrange such a tensor,
/// lib/poplin/Convolution.cpp:2569-2628; packing cannot be undone here.)
/// `what` names the operand in the message.
void requirePackedFor(const mxconv_plan *plan, const DeviceTensor &packed,
                      const char *what);
mxconv_stream streamOf(const Stream &s);

} // namespace detail
} // namespace poplin
#endif

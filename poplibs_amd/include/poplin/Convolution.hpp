// poplin's forward-convolution entry points for the MI355X build.
//
// The functions keep the names, argument order and error behaviour of
// PopLibs' include/poplin/Convolution.hpp; what changes is what they act on.
// PopLibs appends vertices to a poplar::Graph and a program::Sequence that an
// Engine runs later; here a tensor is a device buffer (DeviceTensor), a
// "program" is a HIP stream (Stream) on which the work is enqueued at once,
// and the graph / debug-context arguments are gone.  All GPU work goes through
// the C ABI of mxconv.h.
#ifndef poplibs_amd_poplin_Convolution_hpp
#define poplibs_amd_poplin_Convolution_hpp
#include "poplar/OptionFlags.hpp"
#include "poplar/Target.hpp"
#include "poplar/Type.hpp"
#include "poplin/ConvParams.hpp"

#include <cstddef>
#include <cstdint>
#include <iosfwd>
#include <limits>
#include <memory>
#include <tuple>
#include <vector>

struct mxconv_plan;

namespace poplin {

/// Stands in for poplar::program::Sequence: work is enqueued on this stream
/// in call order.  Owns the stream unless constructed from an existing one.
class Stream {
  struct Impl;
  std::shared_ptr<Impl> impl_;

public:
  Stream();                        ///< creates a new stream
  explicit Stream(void *hipStream); ///< wraps an existing hipStream_t
  void *handle() const;
  void synchronize() const; ///< blocks until everything enqueued has run
};

/// FP8 tensors carry a format and a power-of-two scale
/// (poplar::QuarterMetadata in the Poplar SDK).
struct QuarterMetadata {
  enum class Format { F152 = 0, F143 = 1 };
  Format format = Format::F143;
  int scale = 0; ///< value = fp8 * 2^scale, -32..31
  std::uint8_t byte() const {
    return std::uint8_t((unsigned(format) << 7) | (unsigned(scale) & 0x3f));
  }
};

/// Stands in for poplar::Tensor: a reference-counted device buffer with the
/// logical (external) shape of the reference API and a tag for the physical
/// layout it is held in.
class DeviceTensor {
public:
  enum class Layout {
    External,      ///< row-major in the logical shape
    ChannelsLast,  ///< activations [B][field...][C]
    PackedWeights  ///< weights as packed for one plan
  };
  DeviceTensor() = default;
  /// Allocates `bytes` of device memory; throws
  /// poplar::graph_memory_allocation_error when the device is out of memory.
  DeviceTensor(poplar::Type type, std::vector<std::size_t> shape,
               Layout layout, std::size_t bytes);

  bool valid() const { return bool(buffer_); }
  poplar::Type elementType() const { return type_; }
  const std::vector<std::size_t> &shape() const { return shape_; }
  std::size_t numElements() const;
  std::size_t bytes() const { return bytes_; }
  Layout layout() const { return layout_; }
  void *data() const { return buffer_.get(); }
  QuarterMetadata metadata; ///< meaningful for QUARTER tensors only
  /// For a PackedWeights tensor: the plan whose packing it holds (set by
  /// createWeights and preArrangeMatMulInputRHS), so that an update of the
  /// weights can be applied in that packing.
  std::shared_ptr<const void> packedFor;

private:
  poplar::Type type_;
  std::vector<std::size_t> shape_;
  Layout layout_ = Layout::External;
  std::size_t bytes_ = 0;
  std::shared_ptr<void> buffer_;
};

/// Memo of plans keyed by (parameters, options); safe to share between
/// threads (include/poplin/Convolution.hpp:724-733).
class PlanningCache {
public:
  PlanningCache();
  ~PlanningCache();
  std::size_t size() const;
  struct Impl;
  std::unique_ptr<Impl> impl;
};

std::uint64_t getFwdFlops(const ConvParams &params);
/// The backward and weight update passes perform the forward pass's number of
/// operations (lib/poplin/Convolution.cpp:3223-3225); `params` are the
/// forward parameters.
std::uint64_t getBwdFlops(const ConvParams &params);
std::uint64_t getWuFlops(const ConvParams &params);

/// Shader cycles of a pass if every matrix core of the chip retired its peak
/// number of multiply-accumulates in every cycle and nothing else took time
/// (include/poplin/Convolution.hpp:34-77 of PopLibs: MACs / (MACs per cycle and
/// tile x tiles); here MACs / (MACs per cycle and SIMD x 4 SIMDs x 256 CUs)).
/// Per SIMD and cycle gfx950's dense MFMA retires 512 fp16, 1 024 fp8 and 32
/// fp32 MACs - the 2.5 / 5.0 PFLOP/s and 157.3 TFLOP/s peaks at 2.4 GHz.
/// An optimistic figure for efficiency estimates; all three passes perform
/// the forward pass's MACs.  `params` are the forward parameters.
double getFwdPerfectCycleCount(const ConvParams &params);
double getBwdPerfectCycleCount(const ConvParams &params);
double getWuPerfectCycleCount(const ConvParams &params);

/// Weights [convGroups][outChansPerGroup][inChansPerGroup][kernel...], held
/// packed for the plan of (params, options).
DeviceTensor createWeights(const ConvParams &params,
                           const poplar::OptionFlags &options = {},
                           PlanningCache *cache = nullptr);
/// Biases [outChans] in the activations' element type.
DeviceTensor createBiases(const DeviceTensor &activations);
DeviceTensor createBiases(const ConvParams &params,
                          const poplar::OptionFlags &options = {},
                          PlanningCache *cache = nullptr);
/// Input [B][inChans][field...], held channels-last.
DeviceTensor createInput(const ConvParams &params,
                         const poplar::OptionFlags &options = {},
                         PlanningCache *cache = nullptr);
/// Output [B][outChans][outField...], held channels-last.
DeviceTensor createConvOutput(const ConvParams &params,
                              const poplar::OptionFlags &options = {},
                              PlanningCache *cache = nullptr);

/// Convolve `in` with `weights`; returns the output tensor.  Tensors in
/// External layout are converted on the device first.
/// transposeAndFlipWeights: `weights` are the forward pass's
/// [G][params.inChans][params.outChans][kernel...] in the external layout and
/// are passed through weightsTransposeChansFlipXY first - the backward pass
/// with params = getGradientParams(forward parameters).
DeviceTensor convolution(const DeviceTensor &in, const DeviceTensor &weights,
                         const ConvParams &params,
                         bool transposeAndFlipWeights, Stream &prog,
                         const poplar::OptionFlags &options = {},
                         PlanningCache *cache = nullptr);

void convolutionWithOutput(const DeviceTensor &in, const DeviceTensor &weights,
                           const DeviceTensor &out, const ConvParams &params,
                           bool transposeAndFlipWeights, Stream &prog,
                           const poplar::OptionFlags &options = {},
                           PlanningCache *cache = nullptr);

/// weightsOut[g][ci][co][k...] = weightsIn[g][co][ci][flipped k...], both in
/// the external layout (include/poplin/Convolution.hpp:407-412 of PopLibs).
void weightsTransposeChansFlipXY(const DeviceTensor &weightsIn,
                                 const DeviceTensor &weightsOut, Stream &prog);

/// The weights of a fully connected layer arranged for its backward pass
/// (include/poplin/Convolution.hpp:695-711 of PopLibs).  `params` are the
/// backward pass's, a convolution over one field dimension (anything else
/// throws poputil::poplibs_error, lib/poplin/Convolution.cpp:3849-3852);
/// `weights` are the forward pass's [G][params.inChans][params.outChans][k] in
/// the external layout.  Returns [G][params.outChans][params.inChans][k] -
/// the channel axes exchanged, nothing flipped - packed for the plan of
/// (params, options), as createWeights would hand it out.
DeviceTensor fullyConnectedWeightTranspose(
    const DeviceTensor &weights, const ConvParams &params, Stream &prog,
    const poplar::OptionFlags &options = {}, PlanningCache *cache = nullptr);

/// Gradient with respect to the forward weights, [G][Co][Ci][kernel...] in the
/// external layout and the forward output type, from the gradient with
/// respect to the forward output `zDeltas` and the forward input
/// `activations` (include/poplin/Convolution.hpp:460-466 of PopLibs).
/// `params` and `options` are the forward pass's.
DeviceTensor calculateWeightDeltas(const DeviceTensor &zDeltas,
                                   const DeviceTensor &activations,
                                   const ConvParams &params, Stream &prog,
                                   const poplar::OptionFlags &options = {},
                                   PlanningCache *cache = nullptr);

/// weights += scale * weight deltas (include/poplin/Convolution.hpp:516-522
/// of PopLibs).  `weights` are in the external layout or packed (as
/// createWeights returns them); the deltas are formed in the weights' type.
void convolutionWeightUpdate(const DeviceTensor &zDeltas,
                             const DeviceTensor &weights,
                             const DeviceTensor &activations,
                             ConvParams params, float scale, Stream &prog,
                             const poplar::OptionFlags &options = {},
                             PlanningCache *cache = nullptr);

/// biases[c] += scale * sum of zDeltas[b][c][...] over batch and field
/// (include/poplin/Convolution.hpp:556-561 of PopLibs).
void convolutionBiasUpdate(const DeviceTensor &zDeltas,
                           const DeviceTensor &biases, float scale,
                           const poplar::OptionFlags &options, Stream &prog);

void reportWeightUpdatePlanInfo(std::ostream &out, const ConvParams &fwdParams,
                                const poplar::OptionFlags &fwdOptions = {},
                                PlanningCache *cache = nullptr);

/// acts[b][c][...] += biases[c].
void addBias(const DeviceTensor &in, const DeviceTensor &biases, Stream &prog);

void reportPlanInfo(std::ostream &out, const ConvParams &params,
                    const poplar::OptionFlags &options = {},
                    PlanningCache *cache = nullptr);

/// Estimated costs of a plan (include/poplin/Convolution.hpp:590-594 of
/// PopLibs).  cycles: shader-clock cycles of one launch at 2.1 GHz, by the
/// cost model the planner weighs tilings with; `unknown` where that model does
/// not cover the kernel chosen.  memory: bytes of temporary device memory a
/// launch uses.
struct PlanCosts {
  std::size_t cycles;
  std::size_t memory;
  constexpr static std::size_t unknown =
      std::numeric_limits<std::size_t>::max();
  /// (This build's addition.)  The cost model works in microseconds; `cycles`
  /// is that time at this shader clock (MXCONV_ESTIMATE_CLOCK_MHZ), so
  /// cycles / clockMHz gives the microseconds back.
  constexpr static double clockMHz = 2100.0;
};

/// include/poplin/Convolution.hpp:608-611 of PopLibs.
PlanCosts reportPlanEstimatedCosts(const ConvParams &params,
                                   const poplar::OptionFlags &options = {},
                                   PlanningCache *cache = nullptr);

namespace internal {

/// The estimate of reportPlanEstimatedCosts by phase
/// (include/poplin/Convolution.hpp:613-665 of PopLibs; same fields, same
/// text form).  A launch on this device has three of the phases:
/// `rearrangement` (the zero-padded copy of an input whose channels do not
/// fill a vector, the fill of an output field the kernel does not cover),
/// `compute` (the convolution kernel) and `reduction` (the ordered sum of fp32
/// partial tiles where K or the pixels are split over workgroups); the other
/// phases are IPU exchange and tile-level steps and stay zero.
/// parallelSplit: workgroups that run side by side; serialSplit: rounds of
/// them.  The phases' cycles add up to total.cycles; all cycles are
/// PlanCosts::unknown where the model does not cover the kernel.
struct DetailedPlanCosts {
  std::size_t parallelSplit = 1;
  std::size_t serialSplit = 1;
  PlanCosts broadcast = {};
  PlanCosts rearrangement = {};
  PlanCosts dynamicSlice = {};
  PlanCosts transform = {};
  PlanCosts exchange = {};
  PlanCosts tileLevelTransform = {};
  PlanCosts inputsCast = {};
  PlanCosts compute = {};
  PlanCosts reduction = {};
  PlanCosts dynamicUpdate = {};
  PlanCosts addInPlace = {};
  PlanCosts outputCast = {};
  PlanCosts total = {};

  /// Calls fn on each phase in the order above; serialSplitOnly leaves out
  /// the phases that happen once however the convolution is split in series
  /// (broadcast, rearrangement, addInPlace, outputCast).
  template <typename Function>
  void apply(Function fn, bool includeTotal = true,
             bool serialSplitOnly = false) {
    struct Phase {
      PlanCosts DetailedPlanCosts::*member;
      bool oncePerConv;
    };
    static constexpr Phase order[] = {
        {&DetailedPlanCosts::broadcast, true},
        {&DetailedPlanCosts::rearrangement, true},
        {&DetailedPlanCosts::dynamicSlice, false},
        {&DetailedPlanCosts::transform, false},
        {&DetailedPlanCosts::exchange, false},
        {&DetailedPlanCosts::tileLevelTransform, false},
        {&DetailedPlanCosts::inputsCast, false},
        {&DetailedPlanCosts::compute, false},
        {&DetailedPlanCosts::reduction, false},
        {&DetailedPlanCosts::dynamicUpdate, false},
        {&DetailedPlanCosts::addInPlace, true},
        {&DetailedPlanCosts::outputCast, true}};
    for (const Phase &p : order)
      if (!(serialSplitOnly && p.oncePerConv))
        fn(this->*p.member);
    if (includeTotal)
      fn(total);
  }
  template <typename Function>
  void apply(Function fn, bool includeTotal = true,
             bool serialSplitOnly = false) const {
    DetailedPlanCosts copy = *this;
    copy.apply([&fn](PlanCosts &c) { fn(static_cast<const PlanCosts &>(c)); },
               includeTotal, serialSplitOnly);
  }
};

/// "parallelSplit serialSplit" on one line, then "cycles memory" per phase
/// and for the total (lib/poplin/Convolution.cpp:3940-3951 of PopLibs).
std::ostream &operator<<(std::ostream &os, DetailedPlanCosts const &c);
std::istream &operator>>(std::istream &is, DetailedPlanCosts &c);

/// include/poplin/Convolution.hpp:670-676 of PopLibs.
DetailedPlanCosts
reportDetailedPlanEstimatedCosts(const ConvParams &params,
                                 const poplar::OptionFlags &options = {},
                                 PlanningCache *cache = nullptr);

} // namespace internal

/// What poplin::preplan takes for one convolution
/// (include/poplin/Convolution.hpp:386-388 of PopLibs): the target (may be
/// null), the parameters and a pointer to the options.
using ConvPlanParams = std::tuple<const poplar::Target *, const ConvParams,
                                  const poplar::OptionFlags *>;

/// Throws poplar::invalid_option for an unknown key or value.
void convolutionValidateOptions(const poplar::OptionFlags &options);

/// Host <-> device transfer in the tensor's logical (external) layout and
/// element type: the role of Engine::writeTensor / readTensor.  `params` and
/// `options` select the plan whose packing a PackedWeights tensor uses.
void writeTensor(const DeviceTensor &t, const void *host, Stream &prog,
                 const ConvParams &params,
                 const poplar::OptionFlags &options = {},
                 PlanningCache *cache = nullptr);
void readTensor(const DeviceTensor &t, void *host, Stream &prog,
                const ConvParams &params,
                const poplar::OptionFlags &options = {},
                PlanningCache *cache = nullptr);
/// The same for tensors in the External layout, which need no plan.
void writeTensor(const DeviceTensor &t, const void *host, Stream &prog);
void readTensor(const DeviceTensor &t, void *host, Stream &prog);

} // namespace poplin
#endif

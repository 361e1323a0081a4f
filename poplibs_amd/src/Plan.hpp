// The gfx950 tile planner: what replaces PopLibs' IPU convolution planner
// (getPlan, lib/poplin/ConvPlan.cpp:1877-1923) in this build.  A plan fixes
// the kernel, its tile shape and the packed weight layout for one
// (ConvParams, ConvOptions) pair; it is plain host data and creating it
// touches no GPU.
#ifndef poplibs_amd_Plan_hpp
#define poplibs_amd_Plan_hpp
#include "ConvOptions.hpp"
#include "mxconv.h"
#include "kernels.hpp"
#include "poplin/ConvParams.hpp"
#include <cstddef>
#include <memory>
#include <string>
#include <vector>

/// Fixed properties of the one target this library is written for.
namespace gfx950 {
constexpr unsigned numCUs = 256;
constexpr unsigned numXCDs = 8;
constexpr unsigned ldsBytesPerCU = 160 * 1024;
constexpr unsigned wavefrontSize = 64;
} // namespace gfx950

struct mxconv_plan {
  enum class Kernel { GENERIC, IGEMM, DEPTHWISE };

  poplin::ConvParams params;    // as given by the caller
  poplin::ConvParams canonical; // ConvParams::canonicalize() of it
  poplin::ConvOptions options;
  bool zeroConv = false;
  Kernel kernel = Kernel::GENERIC;
  std::string reason; // why this kernel was chosen
  // The tilings of the matrix-core kernels the planner weighed for this
  // convolution, with the time each was estimated to take (the role of the
  // reference's per-candidate cost estimates, lib/poplin/ConvPlan.cpp:502-565,
  // reportPlanEstimatedCosts).
  struct Candidate {
    std::string name;
    std::size_t workgroups = 0, perCU = 1, kSteps = 0;
    double rounds = 0, estimateUs = 0;
    bool chosen = false;
  };
  std::vector<Candidate> candidates;

  mxk::GenericDesc generic{};     // always valid: describes `canonical`
  mxk::IgemmDesc igemm{};         // valid when kernel == IGEMM
  // kernel == IGEMM and the streaming small-workgroup kernel serves it (1x1,
  // stride 1, unpadded, few input channels): its descriptor; the packed
  // weights then have its layout.
  bool pointwiseOn = false;
  mxk::PointwiseDesc pointwise{};
  // ... or, for an input of 1 to 4 channels, the kernel that takes a kernel
  // row's pixels as one k-step
  bool thinInputOn = false;
  mxk::ThinInputDesc thinInput{};
  mxk::DepthwiseDesc depthwise{}; // valid when kernel == DEPTHWISE
  // These parameters are the weight update pass of a depthwise layer: the
  // descriptor of that layer's FORWARD convolution, for the kernel that
  // forms the weight deltas straight from the layer's tensors
  // (mxconv_calculate_weight_deltas; the kernel chosen above still serves
  // the parameters as an ordinary convolution).
  // (Both weight-delta kernels are planned only under a weight update pass's
  // options, `pass` TRAINING_WU or FC_TRAINING_WU - what
  // mxconv_weight_update_plan_create sets.)
  bool madeForWeightUpdate = false;
  // ... of a layer without spatial extent (a fully connected layer): the
  // deltas are one matrix product, transpose(dZ) x X, whose result is in
  // weight order as it is - the plan of that product ([Co] x [batch] x [Ci],
  // made by mxconv_weight_update_plan_create).
  std::shared_ptr<const mxconv_plan> weightUpdateProduct;
  bool depthwiseWeightUpdate = false;
  mxk::DepthwiseDesc depthwiseForward{};
  // ... or of a dense layer (any stride): the matrix-core kernel that reads
  // the layer's tensors as they are (mxk::launchWuTap).
  bool denseWeightUpdate = false;
  mxk::WuTapDesc denseForward{};

  // Packed weights of the matrix-core kernel: [G][coPadded][kPadded].
  std::size_t coPadded = 0, kPadded = 0;
  // A convolution over a zero-stuffed input (the backward pass of a strided
  // layer), taken apart: the outputs whose windows meet the same residue of
  // real input rows and columns form one ordinary convolution of the
  // UNdilated input with a sub-kernel - one "phase" each, all in one launch.
  // Empty when the convolution is not run that way.  Each phase's packed
  // weights [G][coPadded][kPadded of the phase] start packedOffset elements
  // into the packed buffer.
  struct IgemmPhase {
    mxk::IgemmDesc d;
    mxk::IgemmTapSelection taps;
    std::size_t packedOffset = 0, kPadded = 0;
  };
  std::vector<IgemmPhase> igemmPhases;
  // The kernel the window applies is a selection of the stored taps (kernel
  // truncation, flips): what the weight packing picks.
  bool kernelSelected = false;
  mxk::IgemmTapSelection igemmTaps{};
  // The output field has zero padding around the convolution's own outputs:
  // the launch fills it with zeros (or the bias) before the kernel writes
  // the inside.
  bool outputPadded = false;
  uint32_t outputPadLoH = 0, outputPadHiH = 0, outputPadLoW = 0,
           outputPadHiW = 0, outputPadLoD = 0, outputPadHiD = 0;

  // Input channels per group as the matrix-core kernel sees them, when that
  // is more than the parameters say (0 otherwise): the channels are padded
  // with zeros to a whole 16-byte vector by a copy into the workspace, at
  // byte offset paddedInputOffset, before every launch.
  std::size_t paddedInputChans = 0, paddedInputOffset = 0;

  // Conv groups run as one by the matrix-core kernels (1: each by itself).
  // A layer of many groups of a few channels (4 or 8 per group of 32, say)
  // fills neither a 16-byte vector of input channels nor a tile of output
  // channels; `convGroupsPerGroup` neighbouring groups are planned, packed
  // and run as ONE group of that many times the channels, whose weights are
  // block-diagonal - the groups' channels are neighbours in the tensors
  // already, so only the weight packing knows.  The role of the reference
  // planner's convGroupsPerGroup (lib/poplin/ConvPlan.cpp, the AMP and SLIC
  // vertices that take several conv groups at once).  The packed-weights
  // buffer then has room behind the packed weights for the block-diagonal
  // weights in external order, `weightExpandElems` elements, which the
  // packing fills first.
  unsigned convGroupsPerGroup = 1;
  std::size_t weightExpandElems = 0;
  // A weight update pass planned for the layer with that many conv groups
  // taken as one (1: as it is): `params` are that fused layer's weight update
  // parameters, the pass forms the fused layer's weight deltas
  // [G / f][f co][f ci][kernel] in its workspace and hands back the f diagonal
  // blocks of every fused group - the layer's own deltas [G][co][ci][kernel].
  unsigned wuGroupsPerGroup = 1;

  std::size_t inputElems = 0, outputElems = 0, weightElems = 0,
              weightPackedElems = 0, biasElems = 0;
  std::size_t workspaceBytes = 0;

  std::size_t inputBytes() const { return inputElems * params.inputType.size(); }
  std::size_t outputBytes() const {
    return outputElems * params.outputType.size();
  }
  std::size_t weightBytes() const {
    return weightElems * params.inputType.size();
  }
  std::size_t weightPackedBytes() const {
    return (weightPackedElems + weightExpandElems) * params.inputType.size();
  }
  std::size_t biasBytes() const { return biasElems * params.outputType.size(); }

  std::string describe() const;
  /// The plan as a complete `planConstraints` document
  /// ({"gfx950": {...}}): given back as that option with the same
  /// parameters it reproduces this plan's kernel, tiling, packing and
  /// workspace exactly, whatever the planner would choose by itself (the
  /// role of getPlanConstraints, lib/poplin/ConvPlan.cpp:1574-1636).
  std::string constraintsJson() const;

  /// Time one launch of this plan is estimated to take on the device, in
  /// microseconds, by the cost model the tilings were weighed with; negative
  /// when the model does not cover the kernel (the generic one).  The role of
  /// estimateConvCost behind reportPlanEstimatedCosts
  /// (lib/poplin/Convolution.cpp:3923-3936).
  double estimatedMicroseconds() const;
  /// The same estimate taken apart, the role of estimateDetailedConvCost
  /// behind reportDetailedPlanEstimatedCosts
  /// (lib/poplin/Convolution.cpp:3953-3962): operands brought into the shape
  /// the kernel takes (the zero-padded copy of an input whose channels are no
  /// whole vector, the fill of a padded output field), the convolution
  /// kernel, and the ordered sum of fp32 partial tiles where K or the pixels
  /// are split over workgroups; workgroups running side by side and rounds
  /// of them.
  struct DetailedEstimate {
    bool known = true; ///< false: the model does not cover the kernel
    double rearrangementUs = 0, computeUs = 0, reductionUs = 0;
    std::size_t rearrangementBytes = 0, reductionBytes = 0;
    std::size_t parallelSplit = 1, serialSplit = 1;
    double totalUs() const {
      return rearrangementUs + computeUs + reductionUs;
    }
  };
  DetailedEstimate detailedEstimate() const;
  /// The shader clock the estimate is converted to cycles with
  /// (MXCONV_ESTIMATE_CLOCK_MHZ): what the chip holds with the matrix cores
  /// of most CUs busy.
  static constexpr double kEstimateClockMHz = MXCONV_ESTIMATE_CLOCK_MHZ;
};

namespace poplin {

/// validateLayerParams (lib/poplin/ConvValidation.cpp:11-70) followed by the
/// kernel and tile choice.  Throws poputil::poplibs_error /
/// poplar::invalid_option.
mxconv_plan makePlan(const ConvParams &params, const ConvOptions &options);

} // namespace poplin
#endif

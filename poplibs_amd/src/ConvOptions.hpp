// Options of a convolution: the string key/value pairs of a
// poplar::OptionFlags, checked as PopLibs checks them
// (lib/poplin/ConvOptions.cpp:105-152, 193-329) and reduced to what the gfx950
// planner uses.
#ifndef poplibs_amd_ConvOptions_hpp
#define poplibs_amd_ConvOptions_hpp
#include "Json.hpp"
#include "poplar/Type.hpp"
#include <string>
#include <utility>
#include <vector>

namespace poplin {

enum class Pass {
  NONE,
  NONE_MATMUL,
  INFERENCE_FWD,
  TRAINING_FWD,
  TRAINING_BWD,
  TRAINING_WU,
  FC_INFERENCE_FWD,
  FC_TRAINING_FWD,
  FC_TRAINING_BWD,
  FC_TRAINING_WU
};
const char *toString(Pass p);

/// What planConstraints may pin for this build.  The PopLibs method names are
/// mapped onto the gfx950 kernels that take over their role.
struct PlanConstraints {
  enum class Method { ANY, AMP, SLIC, HMAC, VMAC, OUTER_PRODUCT };
  Method method = Method::ANY;
  /// Conv groups the matrix-core kernels run as one (the reference's
  /// top-level constraint of that name); 0 = planner's choice.
  unsigned convGroupsPerGroup = 0;
  /// "gfx950" section: force a kernel ("generic", "igemm", "depthwise") and
  /// tile extents; 0 / empty = planner's choice.
  std::string kernel;
  unsigned blockM = 0, blockN = 0, blockK = 0;
  /// Parts the matrix-core kernel cuts K into; 0 = planner's choice.
  unsigned splitK = 0;
  unsigned stages = 0; // LDS stages of the 128-wide igemm tile: 2 or 4
  /// The matrix-core kernel that keeps the input patch in LDS: -1 planner's
  /// choice, 0 never, 1 / 2 whenever it can take the convolution (1: tiles of
  /// 128 or 64 pixels in 32-pixel MFMA blocks; 2: tiles of up to 112 pixels
  /// in 16-pixel blocks, as many equal ones as there are CUs unless blockM
  /// names the height).
  int patch = -1;
  /// Output tile of the depthwise kernel; 0 = planner's choice.
  unsigned tileH = 0, tileW = 0;
  /// The depthwise 3x3 kernel whose persistent workgroups keep a ring of
  /// input rows in LDS: -1 planner's choice, 0 never, 1 whenever it can take
  /// the layer.
  int rowRing = -1;
  /// 64-channel tiles of the output per workgroup of the pointwise streaming
  /// kernel (1 to 4); 0 = planner's choice.
  unsigned chanTiles = 0;
  /// The pointwise streaming kernel (1x1, unit stride, unpadded): -1
  /// planner's choice, 0 never, 1 required (an error where it cannot take the
  /// convolution).
  int pointwise = -1;
  /// The matrix-core kernel for inputs of 1 to 4 channels (a kernel row's
  /// pixels as one k-step, no padded copy of the input): -1 planner's choice
  /// (never with "kernel" or a tile named), 0 never, 1 required.
  int thinInput = -1;
  /// A weight update pass's deltas: -1 planner's choice, 0 through the pass's
  /// own convolution (batch and channels exchanged), 1 by the kernel that
  /// reads the layer's own tensors (an error where none takes the layer), 2
  /// as one matrix product on the transposed deltas (a layer without spatial
  /// extent; an error for any other).
  int weightDeltas = -1;
  std::string text; // the JSON as given, kept for reporting and cache keys
};

class ConvOptions {
public:
  double availableMemoryProportion = .6;
  Pass pass = Pass::NONE;
  poplar::Type partialsType = poplar::FLOAT;
  poplar::Type interTilePartialsType = poplar::FLOAT;
  poplar::Type interIpuPartialsType = poplar::FLOAT;
  PlanConstraints planConstraints;
  std::string planConstraintsOutputFilename;

  ConvOptions() = default;
  /// Throws poplar::invalid_option on an unknown key or a malformed value.
  explicit ConvOptions(
      const std::vector<std::pair<std::string, std::string>> &flags);

  /// Stable text form, used in plan-cache keys.
  std::string key() const;
};

/// Options of the weight update / backward pass of a layer whose forward
/// pass has `fwdOptions`: only `pass` changes, staying within the
/// fully-connected family if it started there
/// (lib/poplin/ConvUtilInternal.cpp:941-970).
ConvOptions getWeightUpdateOptions(ConvOptions fwdOptions);
/// Whether these are the options of a weight update pass.
bool isWeightUpdatePass(Pass p);
/// The file a plan made under `options` dumps its constraints to:
/// planConstraintsOutputFilename + _FWD / _BWD / _WU by the pass (nothing for
/// NONE and NONE_MATMUL) + .json (lib/poplin/ConvPlan.cpp:1642-1666); empty
/// when the option is not set.
std::string getPlanConstraintsOutputFile(const ConvOptions &options);
ConvOptions getGradientOptions(ConvOptions fwdOptions);

} // namespace poplin
#endif

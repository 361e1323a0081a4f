// poplin::multiconv on device buffers: the functions of PopLibs'
// include/poplin/MultiConvolution.hpp with poplar::Graph / Tensor / Sequence
// replaced by DeviceTensor and Stream (see poplin/Convolution.hpp).
//
// Several independent convolutions are handed over together so that they can
// share the device.  PopLibs gives each a disjoint range of IPU tiles; here
// forward passes that run the same matrix-core kernel are issued as one
// launch whose grid is the concatenation of their tiles, so that convolutions
// too small to fill 256 compute units run side by side.  Results are those
// of the single-convolution functions (to rounding, where a convolution's K
// is cut into parts when it runs alone and stays whole in company).
//
// Multi-convolution options (lib/poplin/ConvPlan.cpp:1929-1953 of PopLibs):
// planType = parallel (default) | serial; perConvReservedTiles and
// cycleBackOff are checked and otherwise ignored (they steer the IPU tile
// split).
#ifndef poplibs_amd_poplin_MultiConvolution_hpp
#define poplibs_amd_poplin_MultiConvolution_hpp
#include "poplin/Convolution.hpp"

#include <string>
#include <vector>

namespace poplin {
namespace multiconv {

/// Throws poplar::invalid_option for an unknown multi-convolution option key
/// or value (PopLibs checks them when a multi-plan is made; there is no
/// function of this name there).
void validateOptions(const poplar::OptionFlags &options);

struct CreateTensorArgs {
  ConvParams params;
  poplar::OptionFlags options;
  std::string name;
};

/// The weights / input of convolution `index` of the set, laid out as the
/// single-convolution createWeights / createInput lay them out.
DeviceTensor createWeights(const std::vector<CreateTensorArgs> &args,
                           unsigned weightsIndex,
                           const poplar::OptionFlags &options = {},
                           PlanningCache *cache = nullptr);
DeviceTensor createInput(const std::vector<CreateTensorArgs> &args,
                         unsigned inputIndex,
                         const poplar::OptionFlags &options = {},
                         PlanningCache *cache = nullptr);

struct ConvolutionArgs {
  DeviceTensor inputs;
  DeviceTensor weights;
  ConvParams params;
  poplar::OptionFlags options;
};

/// args[i].weights = weightsIn[i] with channels transposed and every spatial
/// axis flipped; args[i].params are the backward parameters, the tensors are
/// in the external layout.
void weightsTransposeChansFlipXY(std::vector<ConvolutionArgs> &args,
                                 const std::vector<DeviceTensor> &weightsIn,
                                 Stream &prog,
                                 const poplar::OptionFlags &options = {},
                                 PlanningCache *cache = nullptr);

std::vector<DeviceTensor> convolution(const std::vector<ConvolutionArgs> &args,
                                      bool transposeAndFlipWeights,
                                      Stream &prog,
                                      const poplar::OptionFlags &options = {},
                                      PlanningCache *cache = nullptr);

struct CalculateWeightDeltasArgs {
  DeviceTensor zDeltas;
  DeviceTensor activations;
  ConvParams params;
  poplar::OptionFlags options;
};

std::vector<DeviceTensor>
calculateWeightDeltas(const std::vector<CalculateWeightDeltasArgs> &args,
                      Stream &prog, const poplar::OptionFlags &options = {},
                      PlanningCache *cache = nullptr);

struct ConvWeightUpdateArgsScalar {
  DeviceTensor zDeltas;
  DeviceTensor weights;
  DeviceTensor activations;
  float scale;
  ConvParams params;
  poplar::OptionFlags options;
};

void convolutionWeightUpdate(const std::vector<ConvWeightUpdateArgsScalar> &args,
                             Stream &prog,
                             const poplar::OptionFlags &options = {},
                             PlanningCache *cache = nullptr);

} // namespace multiconv
} // namespace poplin
#endif

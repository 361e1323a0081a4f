// Per-dimension index and range algebra of a convolution described by
// poplin::ConvParams; the functions of PopLibs' include/poplin/ConvUtil.hpp.
// Ranges are half-open {begin, end}; an empty range is {0, 0}; ~0U means
// "no such element".
#ifndef poplibs_amd_poplin_ConvUtil_hpp
#define poplibs_amd_poplin_ConvUtil_hpp
#include "poplin/ConvParams.hpp"
#include <cstdint>
#include <utility>

namespace poplin {

using Range = std::pair<unsigned, unsigned>;

unsigned getDilatedSize(unsigned size, unsigned dilation);

unsigned getInputIndex(unsigned dim, unsigned outputIndex, unsigned kernelIndex,
                       const ConvParams &params);
unsigned getKernelIndex(unsigned dim, unsigned outputIndex, unsigned inputIndex,
                        const ConvParams &params);

Range getOutputRangeForKernelIndex(unsigned dim, Range outputRange,
                                   unsigned kernelIndex,
                                   const ConvParams &params);
Range getOutputRangeForInputIndex(unsigned dim, Range outputRange,
                                  unsigned inputIndex,
                                  const ConvParams &params);
Range getOutputRangeForKernelRange(unsigned dim, Range outputRange,
                                   Range kernelIndexRange,
                                   const ConvParams &params);
Range getOutputRangeForInputRange(unsigned dim, Range outputRange,
                                  Range inputRange, const ConvParams &params);

Range getInputRange(unsigned dim, Range outputRange, unsigned kernelIndex,
                    const ConvParams &params);
Range getKernelRange(unsigned dim, Range outputRange, unsigned inputIndex,
                     const ConvParams &params);
Range getInputRange(unsigned dim, Range outputRange, Range kernelIndexRange,
                    const ConvParams &params);
Range getKernelRange(unsigned dim, Range outputRange, Range inputRange,
                     const ConvParams &params);

inline Range getInputRange(unsigned dim, unsigned outputIndex,
                           Range kernelIndexRange, const ConvParams &params) {
  return getInputRange(dim, Range{outputIndex, outputIndex + 1},
                       kernelIndexRange, params);
}
inline Range getInputRange(unsigned dim, unsigned outputIndex,
                           const ConvParams &params) {
  return getInputRange(dim, outputIndex,
                       Range{0, unsigned(params.kernelShape[dim])}, params);
}
inline Range getInputRange(unsigned dim, Range outputRange,
                           const ConvParams &params) {
  return getInputRange(dim, outputRange,
                       Range{0, unsigned(params.kernelShape[dim])}, params);
}

/// Multiply-accumulates of the forward pass, not counting those that land on
/// padding or dilation zeros (lib/poplin/PerformanceEstimation.hpp:1641-1666).
std::uint64_t getNumberOfMACs(const ConvParams &params);

/// True when every output element is zero whatever the data
/// (lib/poplin/ConvUtilInternal.cpp:24-38); expects canonical parameters.
bool isZeroConvolution(const ConvParams &canonicalParams);
/// The canonical all-zero convolution with the same tensor shapes
/// (lib/poplin/ConvUtilInternal.cpp:40-76).
ConvParams getZeroConv(const ConvParams &params);

/// Parameters of the convolution that computes the gradient with respect
/// to the forward pass's input from the gradient with respect to its output
/// and the forward weights with channels transposed and every spatial axis
/// flipped (weightsTransposeChansFlipXY); canonical
/// (lib/poplin/ConvUtil.cpp:728-795).
ConvParams getGradientParams(const ConvParams &params);

/// Parameters of the convolution that computes the gradient with respect to
/// the forward pass's weights: its input are the forward activations with
/// batch and channel axes exchanged, its kernel the gradient with respect to
/// the forward output, its output field the forward kernel; canonical
/// (include/poplin/ConvUtil.hpp:114, lib/poplin/Convolution.cpp:3390-3435).
ConvParams getWeightUpdateParams(const ConvParams &params);

} // namespace poplin
#endif

// Per-dimension index and range algebra for poplin::ConvParams.
//
// The two index functions state the definition (PopLibs
// lib/poplin/ConvUtil.cpp:95-309).  Every range query is then answered from
// that definition by scanning the (output, kernel) index pairs of one
// dimension - the quantity PopLibs falls back to when its interval shortcuts
// are inexact (lib/poplin/ConvUtil.cpp:487-504) - so that the result is the
// tightest half-open range containing every participating index, {0, 0} if
// there is none.  Extents here are a few hundred at most, so the scans cost
// microseconds and planning needs nothing faster.
#include "poplin/ConvUtil.hpp"
#include "poputil/exceptions.hpp"

#include <algorithm>
#include <numeric>

namespace poplin {

namespace {
constexpr unsigned none = ~0U;

struct Dim {
  unsigned size, truncLo, truncHi, dilation, padLo, padHi;
  bool flip;
  unsigned transformedSize() const {
    return padLo + getDilatedSize(size - (truncLo + truncHi), dilation) + padHi;
  }
  /// Index after truncate, dilate, pad, flip; `none` if truncated away
  /// (lib/poplin/ConvUtil.cpp:98-114).
  unsigned forward(unsigned index) const {
    if (index < truncLo || index >= size - truncHi)
      return none;
    const unsigned padded = (index - truncLo) * dilation + padLo;
    return flip ? transformedSize() - 1 - padded : padded;
  }
  /// Inverse of `forward`; `none` for padding and dilation holes
  /// (lib/poplin/ConvUtil.cpp:159-179).
  unsigned backward(unsigned transformed) const {
    const unsigned total = transformedSize();
    const unsigned padded = flip ? total - 1 - transformed : transformed;
    if (padded < padLo || padded >= total - padHi)
      return none;
    const unsigned dilated = padded - padLo;
    if (dilated % dilation != 0)
      return none;
    return dilated / dilation + truncLo;
  }
};

Dim dimOf(const std::vector<std::size_t> &shape,
          const ConvParams::InputTransform &t, unsigned d) {
  return {unsigned(shape[d]), t.truncationLower[d], t.truncationUpper[d],
          t.dilation[d],      t.paddingLower[d],    t.paddingUpper[d],
          bool(t.flip[d])};
}

/// Index into the untransformed convolution result for an output index, or
/// `none` when the output element is padding
/// (lib/poplin/ConvUtil.cpp:248-259).
unsigned convOutIndex(unsigned dim, unsigned outputIndex,
                      const ConvParams &p) {
  const auto &ot = p.outputTransform;
  const unsigned outputSize = unsigned(p.getOutputSize(dim));
  if (outputIndex < ot.paddingLower[dim] ||
      outputIndex >= outputSize - ot.paddingUpper[dim])
    return none;
  return (outputIndex - ot.paddingLower[dim]) * ot.stride[dim] +
         ot.truncationLower[dim];
}

struct Span {
  unsigned lo = none, hi = 0;
  void add(unsigned v) {
    lo = std::min(lo, v);
    hi = std::max(hi, v + 1);
  }
  Range get() const { return lo == none ? Range{0, 0} : Range{lo, hi}; }
};
} // namespace

unsigned getDilatedSize(unsigned size, unsigned dilation) {
  return size == 0 ? 0 : 1 + (size - 1) * dilation;
}

unsigned getInputIndex(unsigned dim, unsigned outputIndex, unsigned kernelIndex,
                       const ConvParams &p) {
  const unsigned paddedKernel =
      dimOf(p.kernelShape, p.kernelTransform, dim).forward(kernelIndex);
  if (paddedKernel == none)
    return none;
  const unsigned convOut = convOutIndex(dim, outputIndex, p);
  if (convOut == none)
    return none;
  return dimOf(p.inputFieldShape, p.inputTransform, dim)
      .backward(paddedKernel + convOut);
}

unsigned getKernelIndex(unsigned dim, unsigned outputIndex, unsigned inputIndex,
                        const ConvParams &p) {
  const unsigned paddedInput =
      dimOf(p.inputFieldShape, p.inputTransform, dim).forward(inputIndex);
  if (paddedInput == none)
    return none;
  const unsigned convOut = convOutIndex(dim, outputIndex, p);
  if (convOut == none || convOut > paddedInput)
    return none;
  const unsigned paddedKernel = paddedInput - convOut;
  const Dim k = dimOf(p.kernelShape, p.kernelTransform, dim);
  if (paddedKernel >= k.transformedSize())
    return none;
  return k.backward(paddedKernel);
}

Range getOutputRangeForKernelIndex(unsigned dim, Range bounds,
                                   unsigned kernelIndex, const ConvParams &p) {
  return getOutputRangeForKernelRange(dim, bounds,
                                      {kernelIndex, kernelIndex + 1}, p);
}

Range getOutputRangeForKernelRange(unsigned dim, Range bounds, Range kernels,
                                   const ConvParams &p) {
  Span out;
  for (unsigned o = bounds.first; o < bounds.second; ++o)
    for (unsigned k = kernels.first; k < kernels.second; ++k)
      if (getInputIndex(dim, o, k, p) != none) {
        out.add(o);
        break;
      }
  return out.get();
}

Range getOutputRangeForInputIndex(unsigned dim, Range bounds,
                                  unsigned inputIndex, const ConvParams &p) {
  Span out;
  for (unsigned o = bounds.first; o < bounds.second; ++o)
    if (getKernelIndex(dim, o, inputIndex, p) != none)
      out.add(o);
  return out.get();
}

Range getOutputRangeForInputRange(unsigned dim, Range bounds, Range inputs,
                                  const ConvParams &p) {
  Span out;
  const unsigned kernelSize = unsigned(p.kernelShape[dim]);
  for (unsigned o = bounds.first; o < bounds.second; ++o)
    for (unsigned k = 0; k != kernelSize; ++k) {
      const unsigned i = getInputIndex(dim, o, k, p);
      if (i != none && i >= inputs.first && i < inputs.second) {
        out.add(o);
        break;
      }
    }
  return out.get();
}

Range getInputRange(unsigned dim, Range outputs, unsigned kernelIndex,
                    const ConvParams &p) {
  return getInputRange(dim, outputs, Range{kernelIndex, kernelIndex + 1}, p);
}

Range getInputRange(unsigned dim, Range outputs, Range kernels,
                    const ConvParams &p) {
  Span in;
  for (unsigned o = outputs.first; o < outputs.second; ++o)
    for (unsigned k = kernels.first; k < kernels.second; ++k) {
      const unsigned i = getInputIndex(dim, o, k, p);
      if (i != none)
        in.add(i);
    }
  return in.get();
}

Range getKernelRange(unsigned dim, Range outputs, unsigned inputIndex,
                     const ConvParams &p) {
  Span k;
  for (unsigned o = outputs.first; o < outputs.second; ++o) {
    const unsigned kernelIndex = getKernelIndex(dim, o, inputIndex, p);
    if (kernelIndex != none)
      k.add(kernelIndex);
  }
  return k.get();
}

Range getKernelRange(unsigned dim, Range outputs, Range inputs,
                     const ConvParams &p) {
  Span ks;
  const unsigned kernelSize = unsigned(p.kernelShape[dim]);
  for (unsigned o = outputs.first; o < outputs.second; ++o)
    for (unsigned k = 0; k != kernelSize; ++k) {
      const unsigned i = getInputIndex(dim, o, k, p);
      if (i != none && i >= inputs.first && i < inputs.second)
        ks.add(k);
    }
  return ks.get();
}

std::uint64_t getNumberOfMACs(const ConvParams &p) {
  std::uint64_t macs = std::uint64_t(p.getNumConvGroups()) * p.getBatchSize() *
                       p.getNumOutputChansPerConvGroup() *
                       p.getNumInputChansPerConvGroup();
  for (unsigned dim = 0; dim != p.getNumFieldDims(); ++dim) {
    const unsigned outputSize = unsigned(p.getOutputSize(dim));
    const unsigned stride = p.outputTransform.stride[dim];
    // For one kernel index, consecutive participating outputs are this far
    // apart (input dilation leaves holes the stride may or may not step over).
    const unsigned macStride =
        std::lcm(stride, p.inputTransform.dilation[dim]) / stride;
    std::uint64_t fieldMACs = 0;
    const unsigned kBegin = p.kernelTransform.truncationLower[dim];
    const unsigned kEnd =
        unsigned(p.kernelShape[dim]) - p.kernelTransform.truncationUpper[dim];
    for (unsigned k = kBegin; k < kEnd; ++k) {
      const Range r = getOutputRangeForKernelIndex(dim, {0, outputSize}, k, p);
      fieldMACs += (r.second - r.first + macStride - 1) / macStride;
    }
    macs *= fieldMACs;
  }
  return macs;
}

bool isZeroConvolution(const ConvParams &p) {
  if (p.inputChannelsPerConvGroup == 0 || p.outputChannelsPerConvGroup == 0 ||
      p.batchSize == 0 || p.numConvGroups == 0)
    return true;
  for (unsigned dim = 0; dim != p.getNumFieldDims(); ++dim)
    if (p.outputTransform.paddingLower[dim] +
            p.outputTransform.paddingUpper[dim] ==
        p.getOutputSize(dim))
      return true;
  return false;
}

ConvParams getGradientParams(const ConvParams &params) {
  const ConvParams p = params.canonicalize();
  const unsigned numFieldDims = unsigned(p.getNumFieldDims());
  // A "valid" forward convolution is a "full" one going backwards: a valid
  // one with (kernel size - 1) of padding, on top of what the forward pass
  // truncated from its output.
  auto inputPaddingLower = p.outputTransform.truncationLower;
  auto inputPaddingUpper = p.outputTransform.truncationUpper;
  for (unsigned d = 0; d != numFieldDims; ++d) {
    const unsigned k = unsigned(p.getTransformedKernelSize(d));
    inputPaddingLower[d] += k - 1;
    inputPaddingUpper[d] += k - 1;
  }
  // The caller flips the weights in every spatial axis, which swaps the
  // kernel's lower and upper truncation / padding.  An input flipped in the
  // forward pass means an output flipped in the backward pass, i.e. input
  // and kernel both flipped.
  std::vector<bool> flipInput(numFieldDims, false);
  std::vector<bool> flipKernel = p.kernelTransform.flip;
  for (unsigned d = 0; d != numFieldDims; ++d)
    if (p.inputTransform.flip[d]) {
      flipKernel[d] = !flipKernel[d];
      flipInput[d] = !flipInput[d];
    }
  ConvParams::InputTransform inputTransform;
  inputTransform.truncationLower = p.outputTransform.paddingLower;
  inputTransform.truncationUpper = p.outputTransform.paddingUpper;
  inputTransform.dilation = p.outputTransform.stride;
  inputTransform.paddingLower = inputPaddingLower;
  inputTransform.paddingUpper = inputPaddingUpper;
  inputTransform.flip = flipInput;
  ConvParams::InputTransform kernelTransform;
  kernelTransform.truncationLower = p.kernelTransform.truncationUpper;
  kernelTransform.truncationUpper = p.kernelTransform.truncationLower;
  kernelTransform.dilation = p.kernelTransform.dilation;
  kernelTransform.paddingLower = p.kernelTransform.paddingUpper;
  kernelTransform.paddingUpper = p.kernelTransform.paddingLower;
  kernelTransform.flip = flipKernel;
  ConvParams::OutputTransform outputTransform;
  outputTransform.truncationLower = p.inputTransform.paddingLower;
  outputTransform.truncationUpper = p.inputTransform.paddingUpper;
  outputTransform.stride = p.inputTransform.dilation;
  outputTransform.paddingLower = p.inputTransform.truncationLower;
  outputTransform.paddingUpper = p.inputTransform.truncationUpper;
  const ConvParams bwd(p.inputType, p.outputType, p.batchSize,
                       p.getOutputFieldShape(), p.kernelShape,
                       p.getNumOutputChansPerConvGroup(),
                       p.getNumInputChansPerConvGroup(), p.getNumConvGroups(),
                       inputTransform, kernelTransform, outputTransform);
  return bwd.canonicalize();
}

ConvParams getWeightUpdateParams(const ConvParams &params) {
  const ConvParams p = params.canonicalize();
  const unsigned numFieldDims = unsigned(p.getNumFieldDims());
  // The activations keep their transform.  The deltas take the kernel's
  // place: what the forward pass did to its output is undone on them
  // (padding <-> truncation, stride -> dilation), and what it did to its
  // kernel is undone on this convolution's output.
  ConvParams::InputTransform inputTransform = p.inputTransform;
  ConvParams::InputTransform kernelTransform;
  kernelTransform.truncationLower = p.outputTransform.paddingLower;
  kernelTransform.truncationUpper = p.outputTransform.paddingUpper;
  kernelTransform.dilation = p.outputTransform.stride;
  kernelTransform.paddingLower = p.outputTransform.truncationLower;
  kernelTransform.paddingUpper = p.outputTransform.truncationUpper;
  kernelTransform.flip.assign(numFieldDims, false);
  ConvParams::OutputTransform outputTransform;
  outputTransform.truncationLower = p.kernelTransform.paddingLower;
  outputTransform.truncationUpper = p.kernelTransform.paddingUpper;
  outputTransform.stride = p.kernelTransform.dilation;
  outputTransform.paddingLower = p.kernelTransform.truncationLower;
  outputTransform.paddingUpper = p.kernelTransform.truncationUpper;
  // A kernel flipped in the forward pass means this pass's output flipped,
  // which is the same as flipping both of its operands.
  for (unsigned d = 0; d != numFieldDims; ++d)
    if (p.kernelTransform.flip[d]) {
      inputTransform.flip[d] = !inputTransform.flip[d];
      kernelTransform.flip[d] = true;
    }
  // Batch and input channels change places; the forward output field is the
  // kernel, the forward kernel the output field.
  const ConvParams wu(p.inputType, p.outputType,
                      p.getNumInputChansPerConvGroup(), p.inputFieldShape,
                      p.getOutputFieldShape(), p.getBatchSize(),
                      p.getNumOutputChansPerConvGroup(), p.getNumConvGroups(),
                      inputTransform, kernelTransform, outputTransform);
  return wu.canonicalize();
}

ConvParams getZeroConv(const ConvParams &params) {
  // Truncate input and kernel to nothing, pad each back to one zero, convolve
  // to a single element, truncate it away and pad the output to full size.
  ConvParams z = params;
  const auto n = params.getNumFieldDims();
  const std::vector<unsigned> zeros(n, 0), ones(n, 1);
  auto whole = [](const std::vector<std::size_t> &shape) {
    return std::vector<unsigned>(shape.begin(), shape.end());
  };
  z.inputTransform = ConvParams::InputTransform(
      zeros, whole(params.inputFieldShape), ones, ones, zeros,
      std::vector<bool>(n, false));
  z.kernelTransform = ConvParams::InputTransform(
      zeros, whole(params.kernelShape), ones, ones, zeros,
      std::vector<bool>(n, false));
  z.outputTransform = ConvParams::OutputTransform(
      zeros, ones, ones, zeros, whole(params.getOutputFieldShape()));
  return z;
}

} // namespace poplin

// poplin::ConvParams for the MI355X build: the same descriptor, field names
// and member functions as PopLibs' include/poplin/ConvParams.hpp:16-224, so
// that code written against that header compiles against this one.
#ifndef poplibs_amd_poplin_ConvParams_hpp
#define poplibs_amd_poplin_ConvParams_hpp
#include "poplar/Type.hpp"
#include <cstddef>
#include <functional>
#include <iosfwd>
#include <vector>

struct mxconv_params;

namespace poplin {

struct ConvParams {
  /// Applied to the input field and, separately, to the kernel, per spatial
  /// dimension and in this order: truncate, dilate (insert zeros between
  /// elements), zero-pad, flip.
  struct InputTransform {
    std::vector<unsigned> truncationLower, truncationUpper;
    std::vector<unsigned> dilation;
    std::vector<unsigned> paddingLower, paddingUpper;
    std::vector<bool> flip;

    InputTransform() = default;
    /// Identity transform over `numFieldDims` dimensions (dilation 1).
    InputTransform(std::size_t numFieldDims);
    InputTransform(std::vector<unsigned> truncationLower,
                   std::vector<unsigned> truncationUpper,
                   std::vector<unsigned> dilation,
                   std::vector<unsigned> paddingLower,
                   std::vector<unsigned> paddingUpper, std::vector<bool> flip);
    friend bool operator<(const InputTransform &a, const InputTransform &b);
    friend bool operator==(const InputTransform &a, const InputTransform &b);
    friend bool operator!=(const InputTransform &a, const InputTransform &b) {
      return !(a == b);
    }
  };

  /// Applied to the convolution result per spatial dimension and in this
  /// order: truncate, stride (keep every stride-th element), zero-pad.
  struct OutputTransform {
    std::vector<unsigned> truncationLower, truncationUpper;
    std::vector<unsigned> stride;
    std::vector<unsigned> paddingLower, paddingUpper;

    OutputTransform() = default;
    /// Identity transform over `numFieldDims` dimensions (stride 1).
    OutputTransform(std::size_t numFieldDims);
    OutputTransform(std::vector<unsigned> truncationLower,
                    std::vector<unsigned> truncationUpper,
                    std::vector<unsigned> striding,
                    std::vector<unsigned> paddingLower,
                    std::vector<unsigned> paddingUpper);
    friend bool operator<(const OutputTransform &a, const OutputTransform &b);
    friend bool operator==(const OutputTransform &a, const OutputTransform &b);
    friend bool operator!=(const OutputTransform &a, const OutputTransform &b) {
      return !(a == b);
    }
  };

  poplar::Type inputType;
  poplar::Type outputType;
  std::size_t batchSize = 0;
  std::vector<std::size_t> inputFieldShape;
  std::vector<std::size_t> kernelShape;
  std::size_t inputChannelsPerConvGroup = 0;
  std::size_t outputChannelsPerConvGroup = 0;
  std::size_t numConvGroups = 0;
  InputTransform inputTransform;
  InputTransform kernelTransform;
  OutputTransform outputTransform;

  ConvParams() = default;
  ConvParams(poplar::Type dataType, std::size_t batchSize,
             std::vector<std::size_t> inputFieldShape,
             std::vector<std::size_t> kernelShape, std::size_t inputChannels,
             std::size_t outputChannels, std::size_t numConvGroups);
  ConvParams(poplar::Type inputType, poplar::Type outputType,
             std::size_t batchSize, std::vector<std::size_t> inputFieldShape,
             std::vector<std::size_t> kernelShape, std::size_t inputChannels,
             std::size_t outputChannels, std::size_t numConvGroups);
  ConvParams(poplar::Type inputType, poplar::Type outputType,
             std::size_t batchSize, std::vector<std::size_t> inputFieldShape,
             std::vector<std::size_t> kernelShape, std::size_t inputChannels,
             std::size_t outputChannels, std::size_t numConvGroups,
             InputTransform inputTransform, InputTransform kernelTransform,
             OutputTransform outputTransform);

  /// Size of the convolution result before the output transform.
  std::size_t getUntransformedOutputSize(unsigned dim) const;
  std::size_t getOutputSize(unsigned dim) const;
  std::size_t getNumOutputChansPerConvGroup() const {
    return outputChannelsPerConvGroup;
  }
  std::size_t getNumOutputChans() const {
    return outputChannelsPerConvGroup * numConvGroups;
  }
  std::size_t getInputSize(unsigned dim) const { return inputFieldShape[dim]; }
  std::size_t getNumInputChansPerConvGroup() const {
    return inputChannelsPerConvGroup;
  }
  std::size_t getNumInputChans() const {
    return inputChannelsPerConvGroup * numConvGroups;
  }
  std::size_t getNumConvGroups() const { return numConvGroups; }
  std::size_t getNumFieldDims() const { return inputFieldShape.size(); }
  std::vector<std::size_t> getInputFieldShape() const {
    return inputFieldShape;
  }
  std::vector<std::size_t> getKernelShape() const { return kernelShape; }
  std::size_t getBatchSize() const { return batchSize; }
  unsigned getTruncatedInputSize(unsigned dim) const;
  unsigned getTruncatedKernelSize(unsigned dim) const;
  unsigned getTransformedInputSize(unsigned dim) const;
  unsigned getTransformedKernelSize(unsigned dim) const;
  std::vector<std::size_t> getOutputFieldShape() const;

  /// Throws poputil::poplibs_error when the descriptor is inconsistent.
  void validate() const;
  /// Normal form that computes the same result: unused padding / truncation
  /// stripped, stride 1 where one output remains, no flip or dilation on
  /// single-element dimensions; all-zero results map to one "zero conv".
  ConvParams canonicalize() const;

  friend bool operator<(const ConvParams &a, const ConvParams &b);
  friend bool operator==(const ConvParams &a, const ConvParams &b);
  friend bool operator!=(const ConvParams &a, const ConvParams &b) {
    return !(a == b);
  }

  /// Conversions to and from the C ABI's descriptor (mxconv.h).  toC throws
  /// poputil::poplibs_error when there are more field dimensions than the C
  /// struct holds.
  void toC(mxconv_params &out) const;
  static ConvParams fromC(const mxconv_params &in);
};

std::ostream &operator<<(std::ostream &os, const ConvParams &p);
/// Reads the JSON form (keys as the member names above).
std::istream &operator>>(std::istream &is, ConvParams &p);

std::size_t hash_value(const ConvParams::InputTransform &it);
std::size_t hash_value(const ConvParams::OutputTransform &ot);

} // namespace poplin

namespace std {
template <> struct hash<poplin::ConvParams::InputTransform> {
  std::size_t operator()(const poplin::ConvParams::InputTransform &it) const;
};
template <> struct hash<poplin::ConvParams::OutputTransform> {
  std::size_t operator()(const poplin::ConvParams::OutputTransform &ot) const;
};
template <> struct hash<poplin::ConvParams> {
  std::size_t operator()(const poplin::ConvParams &params) const;
};
} // namespace std
#endif

// poplin::ConvParams: construction, validation, size arithmetic, normal form,
// ordering, hashing and text / JSON IO.  Behaviour follows PopLibs'
// lib/poplin/ConvParams.cpp (cited per function); the code is this build's.
#include "poplin/ConvParams.hpp"
#include "Json.hpp"
#include "mxconv.h"
#include "poplin/ConvUtil.hpp"
#include "poputil/exceptions.hpp"

#include <algorithm>
#include <cassert>
#include <istream>
#include <iterator>
#include <ostream>
#include <sstream>
#include <tuple>

namespace poplar {

std::string Type::toString() const {
  switch (id_) {
  case 0:
    return "quarter";
  case 1:
    return "half";
  case 2:
    return "float";
  }
  return "unknown";
}

std::ostream &operator<<(std::ostream &os, const Type &t) {
  return os << t.toString();
}

} // namespace poplar

namespace poplin {

using InputTransform = ConvParams::InputTransform;
using OutputTransform = ConvParams::OutputTransform;
using poputil::poplibs_error;

// ---- construction (lib/poplin/ConvParams.cpp:121-170, 268-290) -----------

InputTransform::InputTransform(std::size_t n)
    : truncationLower(n, 0), truncationUpper(n, 0), dilation(n, 1),
      paddingLower(n, 0), paddingUpper(n, 0), flip(n, false) {}

InputTransform::InputTransform(std::vector<unsigned> tl,
                               std::vector<unsigned> tu,
                               std::vector<unsigned> dil,
                               std::vector<unsigned> pl,
                               std::vector<unsigned> pu, std::vector<bool> f)
    : truncationLower(std::move(tl)), truncationUpper(std::move(tu)),
      dilation(std::move(dil)), paddingLower(std::move(pl)),
      paddingUpper(std::move(pu)), flip(std::move(f)) {}

OutputTransform::OutputTransform(std::size_t n)
    : truncationLower(n, 0), truncationUpper(n, 0), stride(n, 1),
      paddingLower(n, 0), paddingUpper(n, 0) {}

OutputTransform::OutputTransform(std::vector<unsigned> tl,
                                 std::vector<unsigned> tu,
                                 std::vector<unsigned> s,
                                 std::vector<unsigned> pl,
                                 std::vector<unsigned> pu)
    : truncationLower(std::move(tl)), truncationUpper(std::move(tu)),
      stride(std::move(s)), paddingLower(std::move(pl)),
      paddingUpper(std::move(pu)) {}

ConvParams::ConvParams(poplar::Type inType, poplar::Type outType,
                       std::size_t batch, std::vector<std::size_t> field,
                       std::vector<std::size_t> kernel, std::size_t inChans,
                       std::size_t outChans, std::size_t groups,
                       InputTransform inT, InputTransform kT,
                       OutputTransform outT)
    : inputType(inType), outputType(outType), batchSize(batch),
      inputFieldShape(std::move(field)), kernelShape(std::move(kernel)),
      inputChannelsPerConvGroup(inChans), outputChannelsPerConvGroup(outChans),
      numConvGroups(groups), inputTransform(std::move(inT)),
      kernelTransform(std::move(kT)), outputTransform(std::move(outT)) {}

ConvParams::ConvParams(poplar::Type inType, poplar::Type outType,
                       std::size_t batch, std::vector<std::size_t> field,
                       std::vector<std::size_t> kernel, std::size_t inChans,
                       std::size_t outChans, std::size_t groups)
    : inputType(inType), outputType(outType), batchSize(batch),
      inputFieldShape(std::move(field)), kernelShape(std::move(kernel)),
      inputChannelsPerConvGroup(inChans), outputChannelsPerConvGroup(outChans),
      numConvGroups(groups), inputTransform(inputFieldShape.size()),
      kernelTransform(inputFieldShape.size()),
      outputTransform(inputFieldShape.size()) {}

ConvParams::ConvParams(poplar::Type dataType, std::size_t batch,
                       std::vector<std::size_t> field,
                       std::vector<std::size_t> kernel, std::size_t inChans,
                       std::size_t outChans, std::size_t groups)
    : ConvParams(dataType, dataType, batch, std::move(field),
                 std::move(kernel), inChans, outChans, groups) {}

// ---- ordering (lib/poplin/ConvParams.cpp:69-119) --------------------------

static auto tie(const InputTransform &t) {
  return std::tie(t.truncationLower, t.truncationUpper, t.dilation,
                  t.paddingLower, t.paddingUpper, t.flip);
}
static auto tie(const OutputTransform &t) {
  return std::tie(t.truncationLower, t.truncationUpper, t.stride,
                  t.paddingLower, t.paddingUpper);
}
bool operator<(const InputTransform &a, const InputTransform &b) {
  return tie(a) < tie(b);
}
bool operator==(const InputTransform &a, const InputTransform &b) {
  return tie(a) == tie(b);
}
bool operator<(const OutputTransform &a, const OutputTransform &b) {
  return tie(a) < tie(b);
}
bool operator==(const OutputTransform &a, const OutputTransform &b) {
  return tie(a) == tie(b);
}
static auto tie(const ConvParams &p) {
  return std::tie(p.inputType, p.outputType, p.batchSize, p.inputFieldShape,
                  p.kernelShape, p.inputChannelsPerConvGroup,
                  p.outputChannelsPerConvGroup, p.numConvGroups,
                  p.inputTransform, p.kernelTransform, p.outputTransform);
}
bool operator<(const ConvParams &a, const ConvParams &b) {
  return tie(a) < tie(b);
}
bool operator==(const ConvParams &a, const ConvParams &b) {
  return tie(a) == tie(b);
}

// ---- size arithmetic (lib/poplin/ConvParams.cpp:631-698) ------------------

static unsigned transformedSize(const std::vector<std::size_t> &shape,
                                const InputTransform &t, unsigned dim) {
  const unsigned truncated =
      unsigned(shape[dim]) - (t.truncationLower[dim] + t.truncationUpper[dim]);
  return t.paddingLower[dim] + getDilatedSize(truncated, t.dilation[dim]) +
         t.paddingUpper[dim];
}

unsigned ConvParams::getTruncatedInputSize(unsigned dim) const {
  return unsigned(inputFieldShape[dim]) - (inputTransform.truncationLower[dim] +
                                           inputTransform.truncationUpper[dim]);
}
unsigned ConvParams::getTruncatedKernelSize(unsigned dim) const {
  return unsigned(kernelShape[dim]) - (kernelTransform.truncationLower[dim] +
                                       kernelTransform.truncationUpper[dim]);
}
unsigned ConvParams::getTransformedInputSize(unsigned dim) const {
  return transformedSize(inputFieldShape, inputTransform, dim);
}
unsigned ConvParams::getTransformedKernelSize(unsigned dim) const {
  return transformedSize(kernelShape, kernelTransform, dim);
}
std::size_t ConvParams::getUntransformedOutputSize(unsigned dim) const {
  return std::size_t(getTransformedInputSize(dim)) + 1 -
         getTransformedKernelSize(dim);
}
std::size_t ConvParams::getOutputSize(unsigned dim) const {
  const auto truncated = getUntransformedOutputSize(dim) -
                         (outputTransform.truncationLower[dim] +
                          outputTransform.truncationUpper[dim]);
  const auto stride = outputTransform.stride[dim];
  return outputTransform.paddingLower[dim] + (truncated + stride - 1) / stride +
         outputTransform.paddingUpper[dim];
}
std::vector<std::size_t> ConvParams::getOutputFieldShape() const {
  std::vector<std::size_t> shape(inputFieldShape.size());
  for (unsigned dim = 0; dim != shape.size(); ++dim)
    shape[dim] = getOutputSize(dim);
  return shape;
}

// ---- validation (lib/poplin/ConvParams.cpp:172-266) -----------------------

static std::string num(std::size_t v) { return std::to_string(v); }

void ConvParams::validate() const {
  const auto numFieldDims = inputFieldShape.size();
  if (kernelShape.size() != numFieldDims)
    throw poplibs_error("Number of kernel field dimensions (" +
                        num(kernelShape.size()) +
                        ") does not match the number of input field "
                        "dimensions (" +
                        num(numFieldDims) + ")");
  for (auto s : outputTransform.stride)
    if (s == 0)
      throw poplibs_error("Stride must be non zero");
  for (auto d : inputTransform.dilation)
    if (d == 0)
      throw poplibs_error("Input dilation must be non zero."
                          " Dilation = 1 results in no dilation");
  for (auto d : kernelTransform.dilation)
    if (d == 0)
      throw poplibs_error("Kernel dilation must be non zero."
                          " Dilation = 1 results in no dilation");
  const std::pair<std::size_t, const char *> ranks[] = {
      {inputTransform.truncationLower.size(), "input truncation (lower)"},
      {inputTransform.truncationUpper.size(), "input truncation (upper)"},
      {inputTransform.dilation.size(), "input dilation"},
      {inputTransform.paddingLower.size(), "input padding (lower)"},
      {inputTransform.paddingUpper.size(), "input padding (upper)"},
      {inputTransform.flip.size(), "input flip"},
      {kernelTransform.truncationLower.size(), "kernel truncation (lower)"},
      {kernelTransform.truncationUpper.size(), "kernel truncation (upper)"},
      {kernelTransform.dilation.size(), "kernel dilation"},
      {kernelTransform.paddingLower.size(), "kernel padding (lower)"},
      {kernelTransform.paddingUpper.size(), "kernel padding (upper)"},
      {kernelTransform.flip.size(), "kernel flip"},
      {outputTransform.truncationLower.size(), "output truncation (lower)"},
      {outputTransform.truncationUpper.size(), "output truncation (upper)"},
      {outputTransform.stride.size(), "stride"},
      {outputTransform.paddingLower.size(), "output padding (lower)"},
      {outputTransform.paddingUpper.size(), "output padding (upper)"},
  };
  for (const auto &r : ranks)
    if (r.first != numFieldDims)
      throw poplibs_error(std::string("Number of ") + r.second +
                          " dimensions (" + num(r.first) +
                          ") does not match the number of field dimensions (" +
                          num(numFieldDims) + ")");
  for (unsigned dim = 0; dim != numFieldDims; ++dim) {
    const auto inTrunc = std::size_t(inputTransform.truncationLower[dim]) +
                         inputTransform.truncationUpper[dim];
    if (inTrunc > inputFieldShape[dim])
      throw poplibs_error("Truncation for dimension " + num(dim) + " (" +
                          num(inTrunc) +
                          ") truncates by more than the size of the field (" +
                          num(inputFieldShape[dim]) + ")");
    const auto kTrunc = std::size_t(kernelTransform.truncationLower[dim]) +
                        kernelTransform.truncationUpper[dim];
    if (kTrunc > kernelShape[dim])
      throw poplibs_error("Truncation for dimension " + num(dim) + " (" +
                          num(kTrunc) +
                          ") truncates by more than the size of the kernel (" +
                          num(kernelShape[dim]) + ")");
    const auto tin = getTransformedInputSize(dim);
    const auto tk = getTransformedKernelSize(dim);
    if (tk == 0)
      throw poplibs_error("Transformed kernel for dimension " + num(dim) +
                          " has zero size");
    if (tin < tk)
      throw poplibs_error("Transformed input size for dimension " + num(dim) +
                          " (" + num(tin) +
                          ") is less than the transformed kernel size (" +
                          num(tk) + ")");
    const auto convOut = getUntransformedOutputSize(dim);
    const auto outTrunc = std::size_t(outputTransform.truncationLower[dim]) +
                          outputTransform.truncationUpper[dim];
    if (outTrunc > convOut)
      throw poplibs_error("Output truncation for dimension " + num(dim) +
                          " (" + num(outTrunc) +
                          ") truncates by more than the size of the "
                          "convolution output (" +
                          num(convOut) + ")");
  }
}

// ---- normal form (lib/poplin/ConvParams.cpp:468-629) ----------------------

ConvParams ConvParams::canonicalize() const {
  validate();
  ConvParams p = *this;
  auto &in = p.inputTransform;
  auto &k = p.kernelTransform;
  auto &out = p.outputTransform;
  for (unsigned dim = 0; dim != getNumFieldDims(); ++dim) {
    const unsigned outSize = unsigned(p.getOutputSize(dim));
    const unsigned kernelSize = unsigned(p.kernelShape[dim]);
    const unsigned inputSize = unsigned(p.inputFieldShape[dim]);

    // Output elements that no (input, kernel) pair reaches are zeros; fold
    // them into the output padding, truncating the elements they replace.
    const Range nonZero =
        getOutputRangeForKernelRange(dim, {0, outSize}, {0, kernelSize}, p);
    if (nonZero.first == nonZero.second)
      return getZeroConv(p);
    const unsigned zerosLower = nonZero.first;
    const unsigned zerosUpper = outSize - nonZero.second;
    if (zerosLower > out.paddingLower[dim]) {
      out.truncationLower[dim] +=
          (zerosLower - out.paddingLower[dim]) * out.stride[dim];
      out.paddingLower[dim] = zerosLower;
    }
    if (zerosUpper > out.paddingUpper[dim]) {
      out.truncationUpper[dim] +=
          (zerosUpper - out.paddingUpper[dim]) * out.stride[dim];
      out.paddingUpper[dim] = zerosUpper;
    }
    // Drop trailing conv-output elements the stride steps over.
    unsigned truncatedConvOut =
        unsigned(p.getUntransformedOutputSize(dim)) -
        (out.truncationLower[dim] + out.truncationUpper[dim]);
    const unsigned ignored = (truncatedConvOut - 1) % out.stride[dim];
    out.truncationUpper[dim] += ignored;
    truncatedConvOut -= ignored;
    if (truncatedConvOut == 1)
      out.stride[dim] = 1;

    // Input elements never read become truncation; the space they occupied
    // after dilation is kept as padding.
    const Range inUsed = getInputRange(dim, {0, outSize}, {0, kernelSize}, p);
    assert(inUsed.first != inUsed.second);
    const unsigned inIgnoredLower = inUsed.first;
    const unsigned inIgnoredUpper = inputSize - inUsed.second;
    if (inIgnoredLower > in.truncationLower[dim]) {
      in.paddingLower[dim] +=
          (inIgnoredLower - in.truncationLower[dim]) * in.dilation[dim];
      in.truncationLower[dim] = inIgnoredLower;
    }
    if (inIgnoredUpper > in.truncationUpper[dim]) {
      in.paddingUpper[dim] +=
          (inIgnoredUpper - in.truncationUpper[dim]) * in.dilation[dim];
      in.truncationUpper[dim] = inIgnoredUpper;
    }

    // The same for kernel elements.
    const Range kUsed = getKernelRange(dim, {0, outSize}, {0, inputSize}, p);
    assert(kUsed.first != kUsed.second);
    const unsigned kIgnoredLower = kUsed.first;
    const unsigned kIgnoredUpper = kernelSize - kUsed.second;
    if (kIgnoredLower > k.truncationLower[dim]) {
      k.paddingLower[dim] +=
          (kIgnoredLower - k.truncationLower[dim]) * k.dilation[dim];
      k.truncationLower[dim] = kIgnoredLower;
    }
    if (kIgnoredUpper > k.truncationUpper[dim]) {
      k.paddingUpper[dim] +=
          (kIgnoredUpper - k.truncationUpper[dim]) * k.dilation[dim];
      k.truncationUpper[dim] = kIgnoredUpper;
    }

    // Padding present on both operands at the same (post-flip) end cancels.
    unsigned &kPadLo = k.flip[dim] ? k.paddingUpper[dim] : k.paddingLower[dim];
    unsigned &kPadHi = k.flip[dim] ? k.paddingLower[dim] : k.paddingUpper[dim];
    unsigned &inPadLo =
        in.flip[dim] ? in.paddingUpper[dim] : in.paddingLower[dim];
    unsigned &inPadHi =
        in.flip[dim] ? in.paddingLower[dim] : in.paddingUpper[dim];
    unsigned excess =
        std::min({inPadLo, kPadLo, p.getTransformedKernelSize(dim) - 1});
    inPadLo -= excess;
    kPadLo -= excess;
    excess = std::min({inPadHi, kPadHi, p.getTransformedKernelSize(dim) - 1});
    inPadHi -= excess;
    kPadHi -= excess;

    // Input padding whose results the output truncation discards cancels too.
    excess = std::min({inPadLo, out.truncationLower[dim],
                       unsigned(p.getUntransformedOutputSize(dim) - 1)});
    inPadLo -= excess;
    out.truncationLower[dim] -= excess;
    excess = std::min({inPadHi, out.truncationUpper[dim],
                       unsigned(p.getUntransformedOutputSize(dim) - 1)});
    inPadHi -= excess;
    out.truncationUpper[dim] -= excess;

    // A dimension with at most one surviving element needs neither dilation
    // nor a flip (a flip just swaps its two paddings).
    if (inputSize <= in.truncationLower[dim] + 1 + in.truncationUpper[dim]) {
      in.dilation[dim] = 1;
      if (in.flip[dim]) {
        in.flip[dim] = false;
        std::swap(in.paddingLower[dim], in.paddingUpper[dim]);
      }
    }
    if (kernelSize <= k.truncationLower[dim] + 1 + k.truncationUpper[dim]) {
      k.dilation[dim] = 1;
      if (k.flip[dim]) {
        k.flip[dim] = false;
        std::swap(k.paddingLower[dim], k.paddingUpper[dim]);
      }
    }
    assert(p.getOutputSize(dim) == outSize);
  }
  return p;
}

// ---- text output (lib/poplin/ConvParams.cpp:292-363) ----------------------

template <class C> static void putList(std::ostream &os, const C &c) {
  os << '{';
  bool first = true;
  for (const auto &x : c) {
    if (!first)
      os << ',';
    os << x;
    first = false;
  }
  os << '}';
}

std::ostream &operator<<(std::ostream &os, const ConvParams &p) {
  auto scalar = [&](const char *label, const auto &v) {
    os << "        " << label << v << "\n";
  };
  auto list = [&](const char *label, const auto &v) {
    os << "        " << label;
    putList(os, v);
    os << "\n";
  };
  os << "\n  Params:\n";
  scalar("inputType                  ", p.inputType);
  scalar("outputType                 ", p.outputType);
  scalar("batchSize                  ", p.batchSize);
  scalar("numConvGroups              ", p.numConvGroups);
  list("inputFieldShape            ", p.inputFieldShape);
  list("kernelShape                ", p.kernelShape);
  scalar("inputChannelsPerConvGroup  ", p.inputChannelsPerConvGroup);
  scalar("outputChannelsPerConvGroup ", p.outputChannelsPerConvGroup);
  list("inputTruncationLower       ", p.inputTransform.truncationLower);
  list("inputTruncationUpper       ", p.inputTransform.truncationUpper);
  list("inputDilation              ", p.inputTransform.dilation);
  list("inputPaddingLower          ", p.inputTransform.paddingLower);
  list("inputPaddingUpper          ", p.inputTransform.paddingUpper);
  list("flipInput                  ", p.inputTransform.flip);
  list("kernelTruncationLower      ", p.kernelTransform.truncationLower);
  list("kernelTruncationUpper      ", p.kernelTransform.truncationUpper);
  list("kernelDilation             ", p.kernelTransform.dilation);
  list("kernelPaddingLower         ", p.kernelTransform.paddingLower);
  list("kernelPaddingUpper         ", p.kernelTransform.paddingUpper);
  list("flipKernel                 ", p.kernelTransform.flip);
  list("outputTruncationLower      ", p.outputTransform.truncationLower);
  list("outputTruncationUpper      ", p.outputTransform.truncationUpper);
  list("stride                     ", p.outputTransform.stride);
  list("outputPaddingLower         ", p.outputTransform.paddingLower);
  list("outputPaddingUpper         ", p.outputTransform.paddingUpper);
  list("outputFieldShape           ", p.getOutputFieldShape());
  return os;
}

// ---- JSON input (lib/poplin/ConvParams.cpp:365-458) -----------------------

namespace {
using poplibs_amd::json::Value;

poplar::Type typeFromName(const std::string &name) {
  if (name == "half")
    return poplar::HALF;
  if (name == "float")
    return poplar::FLOAT;
  if (name == "quarter")
    return poplar::QUARTER;
  throw poplibs_error("Unknown element type '" + name + "'");
}

template <class T> void readScalar(const Value &node, const char *key, T &out) {
  if (const Value *v = node.find(key)) {
    unsigned long long u;
    if (!v->asUnsigned(u))
      throw poplibs_error(std::string("'") + key +
                          "' must be a non-negative integer");
    out = static_cast<T>(u);
  }
}

template <class T>
void readVector(const Value &node, const char *key, std::vector<T> &out) {
  const Value *v = node.find(key);
  if (!v)
    return;
  if (!v->isArray())
    throw poplibs_error(std::string("'") + key + "' must be an array");
  std::vector<T> values;
  for (const Value &item : v->items) {
    if constexpr (std::is_same<T, bool>::value) {
      bool b;
      if (!item.asBool(b))
        throw poplibs_error(std::string("'") + key + "' must hold booleans");
      values.push_back(b);
    } else {
      unsigned long long u;
      if (!item.asUnsigned(u))
        throw poplibs_error(std::string("'") + key +
                            "' must hold non-negative integers");
      values.push_back(static_cast<T>(u));
    }
  }
  out = std::move(values);
}

void readInputTransform(const Value &root, const char *key,
                        InputTransform &t) {
  const Value *node = root.find(key);
  if (!node)
    return;
  readVector(*node, "truncationLower", t.truncationLower);
  readVector(*node, "truncationUpper", t.truncationUpper);
  readVector(*node, "dilation", t.dilation);
  readVector(*node, "paddingLower", t.paddingLower);
  readVector(*node, "paddingUpper", t.paddingUpper);
  readVector(*node, "flip", t.flip);
}
} // namespace

std::istream &operator>>(std::istream &is, ConvParams &p) {
  const std::string text((std::istreambuf_iterator<char>(is)),
                         std::istreambuf_iterator<char>());
  Value root;
  try {
    root = poplibs_amd::json::parse(text);
  } catch (const poplibs_amd::json::ParseError &e) {
    throw poplibs_error(e.what());
  }
  if (!root.isObject())
    throw poplibs_error("ConvParams JSON must be an object");
  if (const Value *v = root.find("dataType"))
    p.inputType = p.outputType = typeFromName(v->text);
  if (const Value *v = root.find("inputType"))
    p.inputType = typeFromName(v->text);
  if (const Value *v = root.find("outputType"))
    p.outputType = typeFromName(v->text);
  readScalar(root, "batchSize", p.batchSize);
  readScalar(root, "numConvGroups", p.numConvGroups);
  readScalar(root, "inputChannelsPerConvGroup", p.inputChannelsPerConvGroup);
  readScalar(root, "outputChannelsPerConvGroup", p.outputChannelsPerConvGroup);
  readVector(root, "inputFieldShape", p.inputFieldShape);
  readVector(root, "kernelShape", p.kernelShape);
  if (p.inputFieldShape.size() != p.kernelShape.size())
    throw poplibs_error(
        "Input and kernel must have the same number of dimensions");
  // Transforms absent from the document are the identity.
  const auto n = p.inputFieldShape.size();
  p.inputTransform = InputTransform(n);
  readInputTransform(root, "inputTransform", p.inputTransform);
  p.kernelTransform = InputTransform(n);
  readInputTransform(root, "kernelTransform", p.kernelTransform);
  p.outputTransform = OutputTransform(n);
  if (const Value *node = root.find("outputTransform")) {
    readVector(*node, "truncationLower", p.outputTransform.truncationLower);
    readVector(*node, "truncationUpper", p.outputTransform.truncationUpper);
    readVector(*node, "stride", p.outputTransform.stride);
    readVector(*node, "paddingLower", p.outputTransform.paddingLower);
    readVector(*node, "paddingUpper", p.outputTransform.paddingUpper);
  }
  return is;
}

// ---- hashing (lib/poplin/ConvParams.cpp:460-466, 702-751) -----------------

namespace {
struct Hasher {
  std::size_t seed = 0xcbf29ce484222325ull;
  void add(std::size_t v) {
    seed ^= v + 0x9e3779b97f4a7c15ull + (seed << 6) + (seed >> 2);
  }
  template <class C> void addRange(const C &c) {
    add(c.size());
    for (const auto &x : c)
      add(static_cast<std::size_t>(x));
  }
};
} // namespace

std::size_t hash_value(const InputTransform &it) {
  return std::hash<InputTransform>()(it);
}
std::size_t hash_value(const OutputTransform &ot) {
  return std::hash<OutputTransform>()(ot);
}

// ---- C ABI struct conversion ---------------------------------------------

void ConvParams::toC(mxconv_params &c) const {
  const auto n = inputFieldShape.size();
  if (n > MXCONV_MAX_FIELD_DIMS)
    throw poplibs_error("At most " + num(MXCONV_MAX_FIELD_DIMS) +
                        " field dimensions are supported (got " + num(n) + ")");
  c = mxconv_params{};
  c.input_type = inputType.id();
  c.output_type = outputType.id();
  c.num_field_dims = uint32_t(n);
  c.batch_size = batchSize;
  c.input_channels_per_conv_group = inputChannelsPerConvGroup;
  c.output_channels_per_conv_group = outputChannelsPerConvGroup;
  c.num_conv_groups = numConvGroups;
  auto copyIn = [&](const InputTransform &t, mxconv_input_transform &o) {
    for (unsigned d = 0; d != MXCONV_MAX_FIELD_DIMS; ++d)
      o.dilation[d] = 1;
    for (unsigned d = 0; d != n; ++d) {
      o.truncation_lower[d] = d < t.truncationLower.size() ? t.truncationLower[d] : 0;
      o.truncation_upper[d] = d < t.truncationUpper.size() ? t.truncationUpper[d] : 0;
      o.dilation[d] = d < t.dilation.size() ? t.dilation[d] : 1;
      o.padding_lower[d] = d < t.paddingLower.size() ? t.paddingLower[d] : 0;
      o.padding_upper[d] = d < t.paddingUpper.size() ? t.paddingUpper[d] : 0;
      o.flip[d] = d < t.flip.size() ? t.flip[d] : 0;
    }
  };
  for (unsigned d = 0; d != n; ++d) {
    c.input_field_shape[d] = inputFieldShape[d];
    c.kernel_shape[d] = d < kernelShape.size() ? kernelShape[d] : 0;
  }
  copyIn(inputTransform, c.input_transform);
  copyIn(kernelTransform, c.kernel_transform);
  for (unsigned d = 0; d != MXCONV_MAX_FIELD_DIMS; ++d)
    c.output_transform.stride[d] = 1;
  const auto &ot = outputTransform;
  for (unsigned d = 0; d != n; ++d) {
    c.output_transform.truncation_lower[d] = d < ot.truncationLower.size() ? ot.truncationLower[d] : 0;
    c.output_transform.truncation_upper[d] = d < ot.truncationUpper.size() ? ot.truncationUpper[d] : 0;
    c.output_transform.stride[d] = d < ot.stride.size() ? ot.stride[d] : 1;
    c.output_transform.padding_lower[d] = d < ot.paddingLower.size() ? ot.paddingLower[d] : 0;
    c.output_transform.padding_upper[d] = d < ot.paddingUpper.size() ? ot.paddingUpper[d] : 0;
  }
}

ConvParams ConvParams::fromC(const mxconv_params &c) {
  if (c.num_field_dims > MXCONV_MAX_FIELD_DIMS)
    throw poplibs_error("num_field_dims (" + num(c.num_field_dims) +
                        ") exceeds MXCONV_MAX_FIELD_DIMS");
  if (c.input_type < 0 || c.input_type > 2 || c.output_type < 0 ||
      c.output_type > 2)
    throw poplibs_error("Unknown element type id");
  const unsigned n = c.num_field_dims;
  ConvParams p;
  p.inputType = poplar::Type(c.input_type);
  p.outputType = poplar::Type(c.output_type);
  p.batchSize = c.batch_size;
  p.inputFieldShape.assign(c.input_field_shape, c.input_field_shape + n);
  p.kernelShape.assign(c.kernel_shape, c.kernel_shape + n);
  p.inputChannelsPerConvGroup = c.input_channels_per_conv_group;
  p.outputChannelsPerConvGroup = c.output_channels_per_conv_group;
  p.numConvGroups = c.num_conv_groups;
  auto copyIn = [&](const mxconv_input_transform &i) {
    InputTransform t;
    t.truncationLower.assign(i.truncation_lower, i.truncation_lower + n);
    t.truncationUpper.assign(i.truncation_upper, i.truncation_upper + n);
    t.dilation.assign(i.dilation, i.dilation + n);
    t.paddingLower.assign(i.padding_lower, i.padding_lower + n);
    t.paddingUpper.assign(i.padding_upper, i.padding_upper + n);
    t.flip.resize(n);
    for (unsigned d = 0; d != n; ++d)
      t.flip[d] = i.flip[d] != 0;
    return t;
  };
  p.inputTransform = copyIn(c.input_transform);
  p.kernelTransform = copyIn(c.kernel_transform);
  const auto &o = c.output_transform;
  p.outputTransform.truncationLower.assign(o.truncation_lower, o.truncation_lower + n);
  p.outputTransform.truncationUpper.assign(o.truncation_upper, o.truncation_upper + n);
  p.outputTransform.stride.assign(o.stride, o.stride + n);
  p.outputTransform.paddingLower.assign(o.padding_lower, o.padding_lower + n);
  p.outputTransform.paddingUpper.assign(o.padding_upper, o.padding_upper + n);
  return p;
}

} // namespace poplin

namespace std {

std::size_t hash<poplin::ConvParams::InputTransform>::operator()(
    const poplin::ConvParams::InputTransform &t) const {
  poplin::Hasher h;
  h.addRange(t.truncationLower);
  h.addRange(t.truncationUpper);
  h.addRange(t.dilation);
  h.addRange(t.paddingLower);
  h.addRange(t.paddingUpper);
  h.addRange(t.flip);
  return h.seed;
}

std::size_t hash<poplin::ConvParams::OutputTransform>::operator()(
    const poplin::ConvParams::OutputTransform &t) const {
  poplin::Hasher h;
  h.addRange(t.truncationLower);
  h.addRange(t.truncationUpper);
  h.addRange(t.stride);
  h.addRange(t.paddingLower);
  h.addRange(t.paddingUpper);
  return h.seed;
}

std::size_t
hash<poplin::ConvParams>::operator()(const poplin::ConvParams &p) const {
  poplin::Hasher h;
  h.add(std::size_t(p.inputType.id()));
  h.add(std::size_t(p.outputType.id()));
  h.add(p.batchSize);
  h.addRange(p.inputFieldShape);
  h.addRange(p.kernelShape);
  h.add(p.inputChannelsPerConvGroup);
  h.add(p.outputChannelsPerConvGroup);
  h.add(p.numConvGroups);
  h.add(hash_value(p.inputTransform));
  h.add(hash_value(p.kernelTransform));
  h.add(hash_value(p.outputTransform));
  return h.seed;
}

} // namespace std

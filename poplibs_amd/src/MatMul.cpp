// poplin::matMul* over the C ABI: a multiplication is the convolution
// mxconv_matmul_params describes, run by the kernels a convolution plan picks.
#include "poplin/MatMul.hpp"
#include "popops/ScaledAdd.hpp"
#include "LayerInternal.hpp"
#include "MatMulOptions.hpp"
#include "poplar/exceptions.hpp"
#include "poputil/exceptions.hpp"

#include <ostream>
#include <tuple>

namespace poplin {

using namespace detail;

namespace {

struct Shapes {
  std::size_t g, m, k, n;
};

/// matMulDimChecks / matMulGroupedDimChecks (lib/poplin/MatMul.cpp:406-437)
/// and getConvParams' checks (:240-257).
Shapes checkShapes(const std::vector<std::size_t> &a,
                   const std::vector<std::size_t> &b, bool grouped) {
  const std::size_t rank = grouped ? 3 : 2;
  if (a.size() != rank || b.size() != rank)
    throw poputil::poplibs_error(
        grouped ? "Operand to grouped matrix multiplication is not a matrix."
                : "Operand to matrix multiplication is not a matrix.");
  if (grouped && a[0] != b[0])
    throw poputil::poplibs_error("Group dimensions for the two operands in the "
                                 "grouped multiplication must be the same");
  const std::size_t o = grouped ? 1 : 0;
  if (a[o + 1] != b[o])
    throw poputil::poplibs_error(
        "Second dimension of first operand to matrix multiplication does not "
        "match first dimension of second operand.");
  return {grouped ? a[0] : 1, a[o], a[o + 1], b[o + 1]};
}

poplar::OptionFlags convOptions(const poplar::OptionFlags &options) {
  OptionList list(options.begin(), options.end());
  poplar::OptionFlags conv;
  for (const auto &kv : matMulToConvOptions(list))
    conv.set(kv.first, kv.second);
  return conv;
}

ConvParams convParams(const poplar::Type &in, const poplar::Type &out,
                      const Shapes &s) {
  return ConvParams(in, out, s.m, {1}, {1}, s.k, s.n, s.g);
}

void run(const DeviceTensor &A, const DeviceTensor &B, const DeviceTensor &out,
         bool grouped, Stream &prog, const poplar::OptionFlags &options,
         PlanningCache *cache) {
  const Shapes s = checkShapes(A.shape(), B.shape(), grouped);
  std::vector<std::size_t> expect{s.m, s.n};
  if (grouped)
    expect.insert(expect.begin(), s.g);
  if (out.shape() != expect)
    throw poputil::poplibs_error(
        "Output tensor shape does not match the matrix multiplication");
  if (A.elementType() != B.elementType())
    throw poputil::poplibs_error(
        "Both operands of a matrix multiplication must share an element type");
  for (const DeviceTensor *t : {&A, &out})
    if (t->layout() != DeviceTensor::Layout::External)
      throw poputil::poplibs_error(
          "matMul operands and result are row-major (External layout) tensors");
  if (B.layout() == DeviceTensor::Layout::ChannelsLast)
    throw poputil::poplibs_error(
        "matMul's right-hand side is a row-major tensor or the result of "
        "preArrangeMatMulInputRHS");
  const ConvParams params = convParams(A.elementType(), out.elementType(), s);
  const auto plan = getPlan(params, convOptions(options), cache);
  const mxconv_stream stream = streamOf(prog);

  // With one group the matrices are the convolution's channels-last tensors
  // as they stand; otherwise [g][m][c] <-> [m][g][c] copies go in between.
  DeviceTensor acts = A, result = out;
  if (s.g > 1) {
    acts = DeviceTensor(A.elementType(), A.shape(),
                        DeviceTensor::Layout::ChannelsLast, A.bytes());
    result = DeviceTensor(out.elementType(), out.shape(),
                          DeviceTensor::Layout::ChannelsLast, out.bytes());
    check(mxconv_matmul_lhs_to_internal(plan->plan, A.data(), acts.data(),
                                        stream));
  }
  const std::size_t packedBytes =
      bufferBytes(plan->plan, MXCONV_BUFFER_WEIGHTS_PACKED);
  DeviceTensor packed = B;
  if (B.layout() == DeviceTensor::Layout::External) {
    packed = DeviceTensor(B.elementType(), B.shape(),
                          DeviceTensor::Layout::PackedWeights, packedBytes);
    check(mxconv_matmul_pack_rhs(plan->plan, B.data(), packed.data(), stream));
  } else {
    // (a size match alone would let a buffer arranged for another kernel
    // through: several packed layouts share a size)
    requirePackedFor(plan->plan, B, "right-hand side");
    if (B.bytes() != packedBytes)
      throw poputil::poplibs_error(
          "The pre-arranged right-hand side was made for another "
          "multiplication (other shapes, types or options)");
  }
  const std::size_t wsBytes = bufferBytes(plan->plan, MXCONV_BUFFER_WORKSPACE);
  DeviceTensor workspace;
  if (wsBytes)
    workspace = DeviceTensor(poplar::FLOAT, {wsBytes / 4},
                             DeviceTensor::Layout::External, wsBytes);
  if (A.elementType() == poplar::QUARTER)
    check(mxconv_fwd_quarter(plan->plan, acts.data(), A.metadata.byte(),
                             packed.data(), B.metadata.byte(), nullptr,
                             result.data(), workspace.data(), wsBytes, stream));
  else
    check(mxconv_fwd(plan->plan, acts.data(), packed.data(), nullptr,
                     result.data(), workspace.data(), wsBytes, stream));
  if (s.g > 1)
    check(mxconv_matmul_out_to_external(plan->plan, result.data(), out.data(),
                                        stream));
  // Temporaries are released on return; work enqueued on the stream must
  // have finished with them by then.
  if (s.g > 1 || packed.data() != B.data() || wsBytes)
    prog.synchronize();
}

void accumulate(const DeviceTensor &C, float k, const DeviceTensor &A,
                const DeviceTensor &B, bool grouped, Stream &prog,
                const poplar::OptionFlags &options, PlanningCache *cache) {
  if (C.elementType() == poplar::QUARTER)
    throw poputil::poplibs_error("matMulAcc accumulates into half or float");
  // product = A * B in C's type, then C += k * product
  // (lib/poplin/MatMul.cpp:511-518).
  DeviceTensor product(C.elementType(), C.shape(),
                       DeviceTensor::Layout::External, C.bytes());
  run(A, B, product, grouped, prog, options, cache);
  popops::scaledAddTo(C, product, k, prog);
  prog.synchronize(); // the product is released on return
}

DeviceTensor preArrange(const std::vector<std::size_t> &aShape,
                        const DeviceTensor &B, bool grouped, Stream &prog,
                        const poplar::Type &outputType,
                        const poplar::OptionFlags &options,
                        PlanningCache *cache) {
  if (B.layout() == DeviceTensor::Layout::PackedWeights)
    return B;
  const Shapes s = checkShapes(aShape, B.shape(), grouped);
  const auto plan = getPlan(convParams(B.elementType(), outputType, s),
                            convOptions(options), cache);
  DeviceTensor packed(B.elementType(), B.shape(),
                      DeviceTensor::Layout::PackedWeights,
                      bufferBytes(plan->plan, MXCONV_BUFFER_WEIGHTS_PACKED));
  packed.metadata = B.metadata;
  packed.packedFor = plan;
  check(mxconv_matmul_pack_rhs(plan->plan, B.data(), packed.data(),
                               streamOf(prog)));
  return packed;
}

DeviceTensor allocate(const poplar::Type &type,
                      const std::vector<std::size_t> &shape) {
  std::size_t elems = 1;
  for (auto d : shape)
    elems *= d;
  return DeviceTensor(type, shape, DeviceTensor::Layout::External,
                      elems * type.size());
}

DeviceTensor multiply(const DeviceTensor &A, const DeviceTensor &B,
                      bool grouped, Stream &prog, const poplar::Type &outputType,
                      const poplar::OptionFlags &options,
                      PlanningCache *cache) {
  const Shapes s = checkShapes(A.shape(), B.shape(), grouped);
  std::vector<std::size_t> shape{s.m, s.n};
  if (grouped)
    shape.insert(shape.begin(), s.g);
  DeviceTensor out = allocate(outputType, shape);
  run(A, B, out, grouped, prog, options, cache);
  return out;
}

void report(std::ostream &os, const poplar::Type &inputType,
            const poplar::Type &outputType,
            const std::vector<std::size_t> &aShape,
            const std::vector<std::size_t> &bShape, bool grouped,
            const poplar::OptionFlags &options, PlanningCache *cache) {
  const Shapes s = checkShapes(aShape, bShape, grouped);
  reportPlanInfo(os, convParams(inputType, outputType, s), convOptions(options),
                 cache);
}

} // namespace

DeviceTensor matMul(const DeviceTensor &A, const DeviceTensor &B, Stream &prog,
                    const poplar::OptionFlags &options, PlanningCache *cache) {
  return multiply(A, B, false, prog, A.elementType(), options, cache);
}
DeviceTensor matMul(const DeviceTensor &A, const DeviceTensor &B, Stream &prog,
                    const poplar::Type &outputType,
                    const poplar::OptionFlags &options, PlanningCache *cache) {
  return multiply(A, B, false, prog, outputType, options, cache);
}
void matMulWithOutput(const DeviceTensor &A, const DeviceTensor &B,
                      const DeviceTensor &out, Stream &prog,
                      const poplar::OptionFlags &options,
                      PlanningCache *cache) {
  run(A, B, out, false, prog, options, cache);
}
DeviceTensor matMulGrouped(const DeviceTensor &A, const DeviceTensor &B,
                           Stream &prog, const poplar::Type &outputType,
                           const poplar::OptionFlags &options,
                           PlanningCache *cache) {
  return multiply(A, B, true, prog, outputType, options, cache);
}
void matMulGroupedWithOutput(const DeviceTensor &A, const DeviceTensor &B,
                             const DeviceTensor &out, Stream &prog,
                             const poplar::OptionFlags &options,
                             PlanningCache *cache) {
  run(A, B, out, true, prog, options, cache);
}

void matMulAcc(const DeviceTensor &C, float k, const DeviceTensor &A,
               const DeviceTensor &B, Stream &prog,
               const poplar::OptionFlags &options, PlanningCache *cache) {
  accumulate(C, k, A, B, false, prog, options, cache);
}
void matMulGroupedAcc(const DeviceTensor &C, float k, const DeviceTensor &A,
                      const DeviceTensor &B, Stream &prog,
                      const poplar::OptionFlags &options,
                      PlanningCache *cache) {
  accumulate(C, k, A, B, true, prog, options, cache);
}

DeviceTensor transposeGroupedMatrix(const DeviceTensor &A, Stream &prog) {
  const auto &shape = A.shape();
  if (shape.size() != 2 && shape.size() != 3)
    throw poputil::poplibs_error("Operand to transposition is not a matrix.");
  if (A.layout() != DeviceTensor::Layout::External)
    throw poputil::poplibs_error(
        "transposeGroupedMatrix takes a row-major (External layout) tensor");
  const std::size_t o = shape.size() - 2;
  std::vector<std::size_t> transposed = shape;
  std::swap(transposed[o], transposed[o + 1]);
  DeviceTensor out(A.elementType(), transposed, DeviceTensor::Layout::External,
                   A.bytes());
  out.metadata = A.metadata;
  check(mxconv_transpose_grouped_matrix(A.elementType().id(),
                                        o ? shape[0] : 1, shape[o],
                                        shape[o + 1], A.data(), out.data(),
                                        streamOf(prog)));
  return out;
}

DeviceTensor preArrangeMatMulInputRHS(const std::vector<std::size_t> &aShape,
                                      const DeviceTensor &B, Stream &prog,
                                      const poplar::Type &outputType,
                                      const poplar::OptionFlags &options,
                                      PlanningCache *cache) {
  return preArrange(aShape, B, false, prog, outputType, options, cache);
}
DeviceTensor preArrangeMatMulGroupedInputRHS(
    const std::vector<std::size_t> &aShape, const DeviceTensor &B,
    Stream &prog, const poplar::Type &outputType,
    const poplar::OptionFlags &options, PlanningCache *cache) {
  return preArrange(aShape, B, true, prog, outputType, options, cache);
}

void matMulReportPlan(std::ostream &out, const poplar::Type &inputType,
                      const poplar::Type &outputType,
                      const std::vector<std::size_t> &aShape,
                      const std::vector<std::size_t> &bShape,
                      const poplar::OptionFlags &options,
                      PlanningCache *cache) {
  report(out, inputType, outputType, aShape, bShape, false, options, cache);
}
void matMulGroupedReportPlan(std::ostream &out, const poplar::Type &inputType,
                             const poplar::Type &outputType,
                             const std::vector<std::size_t> &aShape,
                             const std::vector<std::size_t> &bShape,
                             const poplar::OptionFlags &options,
                             PlanningCache *cache) {
  report(out, inputType, outputType, aShape, bShape, true, options, cache);
}

DeviceTensor createMatMulInputLHS(const poplar::Type &dataType,
                                  const std::vector<std::size_t> &aShape,
                                  const std::vector<std::size_t> &bShape,
                                  const poplar::OptionFlags &options,
                                  PlanningCache *) {
  checkShapes(aShape, bShape, false);
  matmulValidateOptions(options);
  return allocate(dataType, aShape);
}
DeviceTensor createMatMulInputRHS(const poplar::Type &dataType,
                                  const std::vector<std::size_t> &aShape,
                                  const std::vector<std::size_t> &bShape,
                                  const poplar::OptionFlags &options,
                                  PlanningCache *) {
  checkShapes(aShape, bShape, false);
  matmulValidateOptions(options);
  return allocate(dataType, bShape);
}
DeviceTensor createMatMulGroupedInputLHS(const poplar::Type &dataType,
                                         const std::vector<std::size_t> &aShape,
                                         const std::vector<std::size_t> &bShape,
                                         const poplar::OptionFlags &options,
                                         PlanningCache *) {
  checkShapes(aShape, bShape, true);
  matmulValidateOptions(options);
  return allocate(dataType, aShape);
}
DeviceTensor createMatMulGroupedInputRHS(const poplar::Type &dataType,
                                         const std::vector<std::size_t> &aShape,
                                         const std::vector<std::size_t> &bShape,
                                         const poplar::OptionFlags &options,
                                         PlanningCache *) {
  checkShapes(aShape, bShape, true);
  matmulValidateOptions(options);
  return allocate(dataType, bShape);
}

DeviceTensor createMatMulOutput(const poplar::Type &,
                                const poplar::Type &outputType,
                                const std::vector<std::size_t> &aShape,
                                const std::vector<std::size_t> &bShape,
                                const poplar::OptionFlags &options,
                                PlanningCache *) {
  const Shapes s = checkShapes(aShape, bShape, false);
  matmulValidateOptions(options);
  return allocate(outputType, {s.m, s.n});
}
DeviceTensor createMatMulGroupedOutput(const poplar::Type &,
                                       const poplar::Type &outputType,
                                       const std::vector<std::size_t> &aShape,
                                       const std::vector<std::size_t> &bShape,
                                       const poplar::OptionFlags &options,
                                       PlanningCache *) {
  const Shapes s = checkShapes(aShape, bShape, true);
  matmulValidateOptions(options);
  return allocate(outputType, {s.g, s.m, s.n});
}

bool operator<(const MatMulParams &a, const MatMulParams &b) {
  return std::tie(a.inputType, a.outputType, a.aShape, a.bShape) <
         std::tie(b.inputType, b.outputType, b.aShape, b.bShape);
}

std::set<ConvPlanParams>
matMulGetConvPlanParams(const std::set<MatMulPlanParams> &matmuls,
                        MatMulToConvOptions &matmulToConvOpts) {
  // lib/poplin/MatMul.cpp:344-366: one set of convolution options per
  // distinct options pointer; the map's nodes stay put, so the pointers into
  // it remain valid as it grows.
  std::set<ConvPlanParams> convs;
  for (const auto &matmul : matmuls) {
    const MatMulParams &mm = std::get<1>(matmul);
    const poplar::OptionFlags *options = std::get<2>(matmul);
    if (!options)
      throw poputil::poplibs_error(
          "matMulGetConvPlanParams: null pointer to the options");
    auto res = matmulToConvOpts.emplace(options, poplar::OptionFlags{});
    if (res.second)
      res.first->second = convOptions(*options);
    const bool grouped = mm.aShape.size() == 3;
    const Shapes s = checkShapes(mm.aShape, mm.bShape, grouped);
    convs.emplace(std::get<0>(matmul),
                  convParams(mm.inputType, mm.outputType, s),
                  &res.first->second);
  }
  return convs;
}

void matmulValidateOptions(const poplar::OptionFlags &options) {
  convolutionValidateOptions(convOptions(options));
}

} // namespace poplin

namespace popops {

void scaledAddTo(const poplin::DeviceTensor &A, float scaleA,
                 const poplin::DeviceTensor &B, float scaleB,
                 poplin::Stream &prog) {
  using poplin::DeviceTensor;
  if (A.shape() != B.shape() || A.elementType() != B.elementType() ||
      A.layout() != B.layout() || A.bytes() != B.bytes())
    throw poputil::poplibs_error(
        "scaledAddTo: the tensors differ in shape, type or layout");
  if (A.layout() == DeviceTensor::Layout::PackedWeights)
    throw poputil::poplibs_error("scaledAddTo: packed weights are not summed");
  poplin::detail::check(mxconv_scaled_add_to(
      A.elementType().id(), A.data(), scaleA, B.data(), scaleB,
      A.numElements(), poplin::detail::streamOf(prog)));
}

void scaledAddTo(const poplin::DeviceTensor &A, const poplin::DeviceTensor &B,
                 float scaleB, poplin::Stream &prog) {
  scaledAddTo(A, 1.f, B, scaleB, prog);
}

} // namespace popops

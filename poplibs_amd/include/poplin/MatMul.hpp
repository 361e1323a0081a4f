// poplin matrix multiplication on device buffers: the functions of PopLibs'
// include/poplin/MatMul.hpp, with poplar::Graph / Tensor / Sequence replaced
// by DeviceTensor and Stream (see poplin/Convolution.hpp).  A multiplication
// is planned and run as the equivalent convolution (lib/poplin/MatMul.cpp:
// 236-272), so it uses the same kernels and the same planning cache.
//
// Matrices are row-major device tensors in the External layout: A [m][k],
// B [k][n], C [m][n]; grouped: A [g][m][k], B [g][k][n], C [g][m][n].
// The right-hand side may also be the tensor preArrangeMatMulInputRHS
// returned: B already packed for the plan, which saves the packing pass in
// every multiplication that re-uses it.
//
// Options (include/poplin/MatMul.hpp:33-105 of PopLibs): partialsType,
// fullyConnectedPass, inputRHSIsPreArranged, use128BitConvUnitLoad,
// enableMultiStageReduce, enableFastReduce, remapOutputTensor,
// availableMemoryProportion, planConstraints, gatherOutput,
// disableSRForAMPVertices.  partialsType and planConstraints influence the
// plan; the IPU-only ones are checked and otherwise ignored.
#ifndef poplibs_amd_poplin_MatMul_hpp
#define poplibs_amd_poplin_MatMul_hpp
#include "poplin/Convolution.hpp"

#include <iosfwd>
#include <set>
#include <unordered_map>
#include <vector>

namespace poplin {

/// C = A * B; the result has A's element type, or outputType.
DeviceTensor matMul(const DeviceTensor &A, const DeviceTensor &B, Stream &prog,
                    const poplar::OptionFlags &options = {},
                    PlanningCache *cache = nullptr);
DeviceTensor matMul(const DeviceTensor &A, const DeviceTensor &B, Stream &prog,
                    const poplar::Type &outputType,
                    const poplar::OptionFlags &options = {},
                    PlanningCache *cache = nullptr);
void matMulWithOutput(const DeviceTensor &A, const DeviceTensor &B,
                      const DeviceTensor &out, Stream &prog,
                      const poplar::OptionFlags &options = {},
                      PlanningCache *cache = nullptr);

/// C[g] = A[g] * B[g].
DeviceTensor matMulGrouped(const DeviceTensor &A, const DeviceTensor &B,
                           Stream &prog, const poplar::Type &outputType,
                           const poplar::OptionFlags &options = {},
                           PlanningCache *cache = nullptr);
void matMulGroupedWithOutput(const DeviceTensor &A, const DeviceTensor &B,
                             const DeviceTensor &out, Stream &prog,
                             const poplar::OptionFlags &options = {},
                             PlanningCache *cache = nullptr);

/// C += k * (A * B) (include/poplin/MatMul.hpp:243-250 of PopLibs).
void matMulAcc(const DeviceTensor &C, float k, const DeviceTensor &A,
               const DeviceTensor &B, Stream &prog,
               const poplar::OptionFlags &options = {},
               PlanningCache *cache = nullptr);
void matMulGroupedAcc(const DeviceTensor &C, float k, const DeviceTensor &A,
                      const DeviceTensor &B, Stream &prog,
                      const poplar::OptionFlags &options = {},
                      PlanningCache *cache = nullptr);

/// A [g][rows][cols] -> a new tensor [g][cols][rows].  PopLibs returns a
/// view; tensors here are plain buffers, so this one copies.
DeviceTensor transposeGroupedMatrix(const DeviceTensor &A, Stream &prog);

/// B packed for the multiplication of an aShape matrix by it; pass the
/// result as B.  PopLibs pre-arranges for the TRAINING_BWD pass only and
/// otherwise returns B (lib/poplin/MatMul.cpp:954-979); here packing is the
/// arrangement every pass uses, so it is done for every pass.
DeviceTensor preArrangeMatMulInputRHS(const std::vector<std::size_t> &aShape,
                                      const DeviceTensor &B, Stream &prog,
                                      const poplar::Type &outputType,
                                      const poplar::OptionFlags &options = {},
                                      PlanningCache *cache = nullptr);
DeviceTensor preArrangeMatMulGroupedInputRHS(
    const std::vector<std::size_t> &aShape, const DeviceTensor &B,
    Stream &prog, const poplar::Type &outputType,
    const poplar::OptionFlags &options = {}, PlanningCache *cache = nullptr);

void matMulReportPlan(std::ostream &out, const poplar::Type &inputType,
                      const poplar::Type &outputType,
                      const std::vector<std::size_t> &aShape,
                      const std::vector<std::size_t> &bShape,
                      const poplar::OptionFlags &options = {},
                      PlanningCache *cache = nullptr);
void matMulGroupedReportPlan(std::ostream &out, const poplar::Type &inputType,
                             const poplar::Type &outputType,
                             const std::vector<std::size_t> &aShape,
                             const std::vector<std::size_t> &bShape,
                             const poplar::OptionFlags &options = {},
                             PlanningCache *cache = nullptr);

/// Operands with the given shapes, allocated on the device.
DeviceTensor createMatMulInputLHS(const poplar::Type &dataType,
                                  const std::vector<std::size_t> &aShape,
                                  const std::vector<std::size_t> &bShape,
                                  const poplar::OptionFlags &options = {},
                                  PlanningCache *cache = nullptr);
DeviceTensor createMatMulInputRHS(const poplar::Type &dataType,
                                  const std::vector<std::size_t> &aShape,
                                  const std::vector<std::size_t> &bShape,
                                  const poplar::OptionFlags &options = {},
                                  PlanningCache *cache = nullptr);
DeviceTensor createMatMulGroupedInputLHS(
    const poplar::Type &dataType, const std::vector<std::size_t> &aShape,
    const std::vector<std::size_t> &bShape,
    const poplar::OptionFlags &options = {}, PlanningCache *cache = nullptr);
DeviceTensor createMatMulGroupedInputRHS(
    const poplar::Type &dataType, const std::vector<std::size_t> &aShape,
    const std::vector<std::size_t> &bShape,
    const poplar::OptionFlags &options = {}, PlanningCache *cache = nullptr);

DeviceTensor createMatMulOutput(const poplar::Type &inputType,
                                const poplar::Type &outputType,
                                const std::vector<std::size_t> &aShape,
                                const std::vector<std::size_t> &bShape,
                                const poplar::OptionFlags &options = {},
                                PlanningCache *cache = nullptr);
DeviceTensor createMatMulGroupedOutput(const poplar::Type &inputType,
                                       const poplar::Type &outputType,
                                       const std::vector<std::size_t> &aShape,
                                       const std::vector<std::size_t> &bShape,
                                       const poplar::OptionFlags &options = {},
                                       PlanningCache *cache = nullptr);

/// Throws poplar::invalid_option for an unknown matMul option key or value.
void matmulValidateOptions(const poplar::OptionFlags &options);

/// C = A * B as poplin::preplan takes it (include/poplin/MatMul.hpp:613-631 of
/// PopLibs): aShape [g][m][k] and bShape [g][k][n], or [m][k] and [k][n] for
/// one group.
struct MatMulParams {
  poplar::Type inputType;
  poplar::Type outputType;
  std::vector<std::size_t> aShape;
  std::vector<std::size_t> bShape;
  friend bool operator<(const MatMulParams &a, const MatMulParams &b);
};

/// include/poplin/MatMul.hpp:641-642 of PopLibs; the target may be null.
using MatMulPlanParams = std::tuple<const poplar::Target *, const MatMulParams,
                                    const poplar::OptionFlags *>;
/// The convolution options made from each multiplication's options, kept
/// alive for the pointers in the set matMulGetConvPlanParams returns
/// (include/poplin/MatMul.hpp:648-649 of PopLibs).
using MatMulToConvOptions =
    std::unordered_map<const poplar::OptionFlags *, poplar::OptionFlags>;

/// The convolutions `matmuls` are planned as
/// (include/poplin/MatMul.hpp:661-663 of PopLibs).
std::set<ConvPlanParams>
matMulGetConvPlanParams(const std::set<MatMulPlanParams> &matmuls,
                        MatMulToConvOptions &matmulToConvOpts);

namespace matmul {
/// The older name of the planning cache (include/poplin/MatMul.hpp:682-688 of
/// PopLibs, deprecated there in favour of poplin::PlanningCache).
class PlanningCache : public poplin::PlanningCache {
public:
  poplin::PlanningCache &getImpl() { return *this; }
};
} // namespace matmul

/// The older name for planning matrix multiplications only
/// (include/poplin/MatMul.hpp:665-672 of PopLibs, deprecated there in favour
/// of preplan).
void preplanMatMuls(const std::set<MatMulPlanParams> &matmuls,
                    matmul::PlanningCache &cache);

} // namespace poplin
#endif

// popops::scaledAddTo on device buffers, for the two uses the matrix
// multiplication path has (include/popops/ScaledAdd.hpp:48-61, 216-228 of
// PopLibs): A += scaleB * B, as poplin::matMulAcc applies it, and
// A = scaleA * A + scaleB * B.  Half or float tensors of equal shape and
// type; the expression is evaluated in fp32 and rounded once.
#ifndef poplibs_amd_popops_ScaledAdd_hpp
#define poplibs_amd_popops_ScaledAdd_hpp
#include "poplin/Convolution.hpp"

namespace popops {

void scaledAddTo(const poplin::DeviceTensor &A, const poplin::DeviceTensor &B,
                 float scaleB, poplin::Stream &prog);
void scaledAddTo(const poplin::DeviceTensor &A, float scaleA,
                 const poplin::DeviceTensor &B, float scaleB,
                 poplin::Stream &prog);

} // namespace popops
#endif

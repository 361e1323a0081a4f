// Direct forward convolution for ANY ConvParams: every truncation, dilation,
// padding, flip, stride and output padding, 0 to 4 field dimensions, grouped,
// fp32 / fp16 / fp8 inputs, fp32 accumulation.  It is the correctness anchor
// and the fallback of the planner; the matrix-core and depthwise kernels take
// the shapes that matter for throughput.
//
// One thread computes one output element; threads along a wavefront differ in
// the output channel first, so weight reads ([G][K][Ci][Co], Co fastest) are
// coalesced and activation reads are wave-uniform broadcasts.
//
// The index map is the per-dimension definition of poplin::getInputIndex
// (PopLibs lib/poplin/ConvUtil.cpp:95-268).
#include "device_types.hpp"
#include "kernels.hpp"

namespace mxk {
namespace {

constexpr uint32_t kNone = 0xffffffffu;

__device__ __forceinline__ uint32_t forwardIndex(const DimTransform &t,
                                                 uint32_t index) {
  if (index < t.truncLo || index >= t.size - t.truncHi)
    return kNone;
  const uint32_t padded = (index - t.truncLo) * t.dilation + t.padLo;
  return t.flip ? t.transformedSize - 1 - padded : padded;
}

__device__ __forceinline__ uint32_t backwardIndex(const DimTransform &t,
                                                  uint32_t transformed) {
  const uint32_t padded =
      t.flip ? t.transformedSize - 1 - transformed : transformed;
  if (padded < t.padLo || padded >= t.transformedSize - t.padHi)
    return kNone;
  const uint32_t dilated = padded - t.padLo;
  if (dilated % t.dilation != 0)
    return kNone;
  return dilated / t.dilation + t.truncLo;
}

template <class InT, class OutT>
__global__ __launch_bounds__(256) void genericConvKernel(
    GenericDesc d, const InT *__restrict__ in, const InT *__restrict__ weights,
    const OutT *__restrict__ bias, OutT *__restrict__ out, int inFormat,
    int weightFormat, float scale) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= d.outElems)
    return;
  const uint32_t outChans = d.groups * d.outChansPerGroup;
  const uint32_t inChans = d.groups * d.inChansPerGroup;
  const uint32_t c = uint32_t(tid % outChans);
  uint64_t rest = tid / outChans;
  uint32_t convOut[kMaxDims];
  bool isPadding = false;
  for (int dim = int(d.numDims) - 1; dim >= 0; --dim) {
    const uint32_t o = uint32_t(rest % d.outSize[dim]);
    rest /= d.outSize[dim];
    if (o < d.outPadLo[dim] || o >= d.outSize[dim] - d.outPadHi[dim])
      isPadding = true;
    convOut[dim] = (o - d.outPadLo[dim]) * d.outStride[dim] + d.outTruncLo[dim];
  }
  const uint32_t b = uint32_t(rest);
  const uint32_t g = c / d.outChansPerGroup;
  const uint32_t oc = c % d.outChansPerGroup;

  float acc = 0.0f;
  if (!isPadding) {
    for (uint32_t ke = 0; ke != d.kernelElems; ++ke) {
      // Unflatten the kernel element (row-major, last dimension fastest) and
      // map it, with the output position, to an input position.
      uint32_t krest = ke;
      uint64_t inOffset = 0, inScale = 1;
      bool valid = true;
      for (int dim = int(d.numDims) - 1; dim >= 0; --dim) {
        const uint32_t k = krest % d.kernel[dim].size;
        krest /= d.kernel[dim].size;
        const uint32_t paddedKernel = forwardIndex(d.kernel[dim], k);
        if (paddedKernel == kNone) {
          valid = false;
          break;
        }
        const uint32_t i = backwardIndex(d.in[dim], paddedKernel + convOut[dim]);
        if (i == kNone) {
          valid = false;
          break;
        }
        inOffset += i * inScale;
        inScale *= d.in[dim].size;
      }
      if (!valid)
        continue;
      const InT *inPtr =
          in + (uint64_t(b) * inScale + inOffset) * inChans +
          uint64_t(g) * d.inChansPerGroup;
      const InT *wPtr = weights + (uint64_t(g) * d.kernelElems + ke) *
                                      d.inChansPerGroup * d.outChansPerGroup +
                        oc;
      for (uint32_t ic = 0; ic != d.inChansPerGroup; ++ic)
        acc = fmaf(Load<InT>::at(inPtr, ic, inFormat),
                   Load<InT>::at(wPtr, uint64_t(ic) * d.outChansPerGroup,
                                 weightFormat),
                   acc);
    }
  }
  acc *= scale;
  if (bias)
    acc += Load<OutT>::at(bias, c, 0);
  storeOut(out, tid, acc);
}

template <class InT, class OutT>
hipError_t run(const GenericDesc &d, const void *in, const void *w,
               const void *bias, void *out, const QuarterInfo &q,
               hipStream_t stream) {
  if (d.outElems == 0)
    return hipSuccess;
  const uint64_t blocks = (d.outElems + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((genericConvKernel<InT, OutT>), dim3(uint32_t(blocks)),
                     dim3(256), 0, stream, d, static_cast<const InT *>(in),
                     static_cast<const InT *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out),
                     q.inFormat, q.weightFormat, q.scale);
  return hipGetLastError();
}

} // namespace

hipError_t launchGeneric(const GenericDesc &d, int inType, int outType,
                         const void *in, const void *weights, const void *bias,
                         void *out, const QuarterInfo &q, hipStream_t stream) {
  QuarterInfo unit;
  const QuarterInfo &qi = inType == kQuarter ? q : unit;
  if (inType == kFloat && outType == kFloat)
    return run<float, float>(d, in, weights, bias, out, qi, stream);
  if (inType == kFloat && outType == kHalf)
    return run<float, __half>(d, in, weights, bias, out, qi, stream);
  if (inType == kHalf && outType == kFloat)
    return run<__half, float>(d, in, weights, bias, out, qi, stream);
  if (inType == kHalf && outType == kHalf)
    return run<__half, __half>(d, in, weights, bias, out, qi, stream);
  if (inType == kQuarter && outType == kHalf)
    return run<uint8_t, __half>(d, in, weights, bias, out, qi, stream);
  if (inType == kQuarter && outType == kFloat)
    return run<uint8_t, float>(d, in, weights, bias, out, qi, stream);
  return hipErrorInvalidValue;
}

} // namespace mxk

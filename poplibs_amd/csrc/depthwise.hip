// Depthwise forward convolution (one input and one output channel per group):
// the memory-bound case PopLibs serves with its HorizontalMac vertices
// (lib/poplin/codelets/ConvPartialHorizontalMac.cpp:34-133).  No matrix cores:
// 1.8 flop per byte, so the only thing that matters is moving each input
// element from HBM once and writing each output once.
//
// Channels-last layout: a thread owns 8 consecutive channels (one 16-byte
// vector) of one output pixel, so a wavefront's loads and stores are runs of
// whole 16-byte vectors along the channel axis.  Products are formed and
// accumulated in fp32.
#include "device_types.hpp"
#include "kernels.hpp"

namespace mxk {
namespace {

__device__ __forceinline__ uint32_t xcdSwizzle(uint32_t bid, uint32_t total) {
  const uint32_t xcd = bid & 7u, idx = bid >> 3;
  const uint32_t q = total >> 3, rem = total & 7u;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

union Vec8 {
  uint4 raw;
  __half2 h2[4];
};

template <class OutT> struct StoreVec;
template <> struct StoreVec<__half> {
  static __device__ __forceinline__ void put(__half *p, const float (&v)[8]) {
    Vec8 o;
#pragma unroll
    for (int i = 0; i != 4; ++i)
      o.h2[i] = __floats2half2_rn(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<uint4 *>(p) = o.raw;
  }
};
template <> struct StoreVec<float> {
  static __device__ __forceinline__ void put(float *p, const float (&v)[8]) {
    *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4 *>(p + 4) = float4{v[4], v[5], v[6], v[7]};
  }
};

template <class OutT>
__global__ __launch_bounds__(256) void depthwiseKernel(
    DepthwiseDesc d, uint64_t total, const __half *__restrict__ in,
    const __half *__restrict__ w, const OutT *__restrict__ bias,
    OutT *__restrict__ out) {
  // Each XCD walks one contiguous range of output pixels (whole images when
  // the batch divides by 8), so halo rows shared by neighbouring output rows
  // are re-read from that XCD's L2 rather than from HBM.
  const uint64_t tid =
      uint64_t(xcdSwizzle(blockIdx.x, gridDim.x)) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  const uint32_t vecs = d.channels / 8;
  const uint32_t cv = uint32_t(tid % vecs);
  uint64_t pix = tid / vecs;
  const uint32_t ow = uint32_t(pix % d.outW);
  pix /= d.outW;
  const uint32_t oh = uint32_t(pix % d.outH);
  const uint32_t b = uint32_t(pix / d.outH);

  float acc[8];
#pragma unroll
  for (int i = 0; i != 8; ++i)
    acc[i] = 0.0f;
  const __half *inB = in + size_t(b) * d.inH * d.inW * d.channels + cv * 8;
  const __half *wC = w + cv * 8;
  for (uint32_t kh = 0; kh != d.kH; ++kh) {
    const int ih = int(oh * d.strideH + kh * d.dilH) - d.padH;
    if (ih < int(d.loH) || ih >= int(d.hiH))
      continue;
    for (uint32_t kw = 0; kw != d.kW; ++kw) {
      const int iw = int(ow * d.strideW + kw * d.dilW) - d.padW;
      if (iw < int(d.loW) || iw >= int(d.hiW))
        continue;
      Vec8 x, k;
      x.raw = *reinterpret_cast<const uint4 *>(
          inB + (size_t(ih) * d.inW + iw) * d.channels);
      k.raw = *reinterpret_cast<const uint4 *>(
          wC + size_t(kh * d.kW + kw) * d.channels);
#pragma unroll
      for (int i = 0; i != 4; ++i) {
        const float2 xf = __half22float2(x.h2[i]);
        const float2 kf = __half22float2(k.h2[i]);
        acc[2 * i] = fmaf(xf.x, kf.x, acc[2 * i]);
        acc[2 * i + 1] = fmaf(xf.y, kf.y, acc[2 * i + 1]);
      }
    }
  }
  if (bias) {
#pragma unroll
    for (int i = 0; i != 8; ++i)
      acc[i] += Load<OutT>::at(bias, cv * 8 + i, 0);
  }
  StoreVec<OutT>::put(out + tid * 8, acc);
}

} // namespace

hipError_t launchDepthwise(const DepthwiseDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, hipStream_t stream) {
  if (inType != kHalf || d.channels % 8 != 0)
    return hipErrorInvalidValue;
  const uint64_t total =
      uint64_t(d.batch) * d.outH * d.outW * (d.channels / 8);
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (outType == kHalf)
    hipLaunchKernelGGL(depthwiseKernel<__half>, grid, block, 0, stream, d,
                       total, static_cast<const __half *>(in),
                       static_cast<const __half *>(weightsPacked),
                       static_cast<const __half *>(bias),
                       static_cast<__half *>(out));
  else if (outType == kFloat)
    hipLaunchKernelGGL(depthwiseKernel<float>, grid, block, 0, stream, d, total,
                       static_cast<const __half *>(in),
                       static_cast<const __half *>(weightsPacked),
                       static_cast<const float *>(bias),
                       static_cast<float *>(out));
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

} // namespace mxk

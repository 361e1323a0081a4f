// Depthwise 3x3 forward convolution, the shape that matters most (3x3 taps,
// dilation 1, stride 1 or 2): the same role as depthwise.hip (PopLibs'
// HorizontalMac vertices,
// lib/poplin/codelets/ConvPartialHorizontalMac.cpp:34-133), built from many
// small, short-lived workgroups instead of a few large ones.
//
// What bounds a 1.8 flop/byte kernel is how well its loads use HBM.
// Measured on MI355X, a kernel whose every wave-wide load covers 1 KB of
// consecutive memory, with few registers per thread so that each SIMD holds
// 8 waves, streams 7 TB/s; the same bytes gathered as every second pixel
// reach 5.3 TB/s.  A stride-2 convolution wants every second pixel per
// output, so loading and computing use different thread mappings, with a
// small LDS exchange between them:
//   1. load: thread = (input column, channel vector), channel vector fastest
//      - one 16-byte vector (8 fp16 channels, channels-last) of each input
//      row the workgroup needs, straight down a column.  A wave-wide load is
//      1 KB of one input row.  Pixels outside the input get an out-of-range
//      buffer offset, for which the buffer unit returns zeros;
//   2. the vectors go to LDS (5 rows x 256 vectors = 20 KB at stride 2), one
//      barrier;
//   3. compute: thread = (output row, output column, channel vector) - nine
//      16-byte LDS reads, 72 fp16 x fp16 + fp32 multiply-adds
//      (v_fma_mix_f32), one 16-byte store.
// A workgroup of 256 threads covers floor(256 / vectors per pixel) input
// columns and as many output rows as give every thread an output (2 at
// stride 2 with 96 channels).  Neighbouring workgroups overlap by the kernel
// halo and are numbered so that each XCD works on a contiguous part of the
// image: the overlap is read from that XCD's L2, not twice from HBM.
#include "device_types.hpp"
#include "kernels.hpp"

namespace mxk {
namespace {

// Cache policy of the image loads and the output stores: streaming
// ("non-temporal").  Every byte is used once - the halo a neighbouring
// workgroup reads again still comes from L2, as the HBM counters show - and
// the hint takes a 4 : 1 read / write stream from 65 % to 72 % of the HBM
// peak on this chip; the kernel gains 6 %.
constexpr int kStreaming = 2; // the buffer load's "slc" bit
constexpr int kThreads = 256;
constexpr int kMaxRows = 5; // input rows a workgroup holds
constexpr uint32_t kOutOfRange = 0x80000000u;

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

union Vec8 {
  uintx4 raw;
  __half2 h2[4];
};

struct Dw3x3Args {
  DepthwiseDesc d;
  uint32_t vecs;     // channels / 8
  uint32_t colsIn;   // input columns per workgroup: kThreads / vecs
  uint32_t colsOut;  // output columns per workgroup: (colsIn - 3) / S + 1
  uint32_t rowsOut;  // output rows per workgroup
  uint32_t rowsIn;   // (rowsOut - 1) * S + 3
  uint32_t colBlocks, rowBlocks; // workgroups across / down an image
  uint32_t inBytes;
  FastDiv divVecs, divColBlocks, divRowBlocks, divOutItems;
};

template <class OutT> struct StoreVec;
template <> struct StoreVec<__half> {
  static __device__ __forceinline__ void put(__half *p, const float (&v)[8]) {
    Vec8 o;
#pragma unroll
    for (int i = 0; i != 4; ++i)
      o.h2[i] = roundPairToHalf(v[2 * i], v[2 * i + 1]);
    __builtin_nontemporal_store(o.raw, reinterpret_cast<uintx4 *>(p));
  }
};
template <> struct StoreVec<float> {
  static __device__ __forceinline__ void put(float *p, const float (&v)[8]) {
    *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4 *>(p + 4) = float4{v[4], v[5], v[6], v[7]};
  }
};

__device__ __forceinline__ uintx4 loadVec(__amdgpu_buffer_rsrc_t buffer,
                                          uint32_t offset) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_bit_cast(
      uintx4,
      __builtin_amdgcn_raw_buffer_load_b128(buffer, offset, 0, kStreaming));
#else
  return uintx4{};
#endif
}

/// S: stride (both dimensions), 1 or 2.
template <int S, class OutT>
__global__ __launch_bounds__(kThreads) void depthwise3x3Kernel(
    Dw3x3Args a, const __half *__restrict__ in, const __half *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out) {
  __shared__ __align__(16) uintx4 patch[kMaxRows][kThreads];
  __shared__ __align__(16) uintx4 tapTable[9][kThreads / 3]; // [tap][vector]
  const DepthwiseDesc &d = a.d;

  // Workgroup -> (image, row block, column block), column block fastest; the
  // 8 XCDs, which take workgroups round-robin, each get a contiguous run.
  const uint32_t xcd = blockIdx.x & 7u, idx = blockIdx.x >> 3;
  const uint32_t perXcd = gridDim.x >> 3, rem = gridDim.x & 7u;
  const uint32_t wg = xcd * perXcd + (xcd < rem ? xcd : rem) + idx;
  uint32_t q = a.divColBlocks(wg);
  const uint32_t colBlock = wg - q * a.colBlocks;
  const uint32_t b = a.divRowBlocks(q);
  const uint32_t rowBlock = q - b * a.rowBlocks;

  const uint32_t t = threadIdx.x;
  const uint32_t pixelBytes = d.channels * 2;
  const uint32_t oh0 = rowBlock * a.rowsOut, ow0 = colBlock * a.colsOut;
  const int ih0 = int(oh0 * S) - d.padH, iw0 = int(ow0 * S) - d.padW;

  // 1. + 2.  Thread t holds input column iw0 + t / vecs, channel vector
  // t % vecs: consecutive threads, consecutive memory.
  {
    const __amdgpu_buffer_rsrc_t inBuf = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<__half *>(in), short(0), int(a.inBytes), 0x00020000);
    const int iw = iw0 + int(a.divVecs(t));
    const bool colOk = t < a.colsIn * a.vecs && iw >= int(d.loW) &&
                       iw < int(d.hiW);
    // (image b, row 0, column iw0) + 16 t: may start "before" the image when
    // iw0 < 0; only offsets that end up inside are used.
    const uint32_t origin =
        b * d.inH * d.inW * pixelBytes + uint32_t(iw0) * pixelBytes + t * 16;
    // The kernel taps travel through LDS as well: one global load per tap
    // and channel vector for the whole workgroup instead of nine per thread,
    // which would keep the vector cache busier than the image does.
    uintx4 tapV = {};
    const bool tapLoader = t < 9 * a.vecs;
    uint32_t tapIdx = 0, tapVec = 0;
    if (tapLoader) {
      tapIdx = a.divVecs(t);
      tapVec = t - tapIdx * a.vecs;
      tapV = *reinterpret_cast<const uintx4 *>(w + tapIdx * d.channels +
                                               tapVec * 8);
    }
    uintx4 x[kMaxRows];
#pragma unroll
    for (int y = 0; y != kMaxRows; ++y) {
      const int ih = ih0 + y;
      const bool ok = colOk && uint32_t(y) < a.rowsIn && ih >= int(d.loH) &&
                      ih < int(d.hiH);
      x[y] = loadVec(inBuf, ok ? origin + uint32_t(ih) * d.inW * pixelBytes
                               : kOutOfRange);
    }
#pragma unroll
    for (int y = 0; y != kMaxRows; ++y)
      patch[y][t] = x[y];
    if (tapLoader)
      tapTable[tapIdx][tapVec] = tapV;
  }

  // 3.  Thread t computes output (row r, column j, vector v), v fastest.
  const uint32_t pj = a.divVecs(t);
  const uint32_t v = t - pj * a.vecs;
  const uint32_t r = a.divOutItems(t); // t / (colsOut * vecs)
  const uint32_t j = pj - r * a.colsOut;
  const uint32_t oh = oh0 + r, ow = ow0 + j;
  const bool active = r < a.rowsOut && oh < d.outH && ow < d.outW;
  const uint32_t c = v * 8;
  float acc[8];
#pragma unroll
  for (int e = 0; e != 8; ++e)
    acc[e] = bias ? Load<OutT>::at(bias, c + e, 0) : 0.0f;
  __syncthreads();
  if (!active)
    return;
  Vec8 taps[9];
#pragma unroll
  for (int tap = 0; tap != 9; ++tap)
    taps[tap].raw = tapTable[tap][v];
  const uintx4 *window = &patch[r * S][j * S * a.vecs + v];
#pragma unroll
  for (int kh = 0; kh != 3; ++kh)
#pragma unroll
    for (int kw = 0; kw != 3; ++kw) {
      Vec8 x;
      x.raw = window[kh * kThreads + kw * a.vecs];
      const Vec8 &k = taps[kh * 3 + kw];
#pragma unroll
      for (int e = 0; e != 4; ++e) {
        const float2 xf = __half22float2(x.h2[e]);
        const float2 kf = __half22float2(k.h2[e]);
        acc[2 * e] = fmaf(xf.x, kf.x, acc[2 * e]);
        acc[2 * e + 1] = fmaf(xf.y, kf.y, acc[2 * e + 1]);
      }
    }
  StoreVec<OutT>::put(
      out + ((size_t(b) * d.outH + oh) * d.outW + ow) * d.channels + c, acc);
}

template <int S, class OutT>
hipError_t run(const Dw3x3Args &a, const void *in, const void *w,
               const void *bias, void *out, hipStream_t stream) {
  const uint32_t blocks = a.d.batch * a.rowBlocks * a.colBlocks;
  hipLaunchKernelGGL((depthwise3x3Kernel<S, OutT>), dim3(blocks),
                     dim3(kThreads), 0, stream, a,
                     static_cast<const __half *>(in),
                     static_cast<const __half *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out));
  return hipGetLastError();
}

/// Workgroup shape for `vecs` channel vectors per pixel at stride s; false
/// when a workgroup cannot hold three input columns.
bool shapeFor(const DepthwiseDesc &d, Dw3x3Args &a) {
  const uint32_t s = d.strideH;
  a.vecs = d.channels / 8;
  if (a.vecs == 0 || a.vecs * 9 > kThreads) // 3 columns; 9 taps in one go
    return false;
  a.colsIn = kThreads / a.vecs;
  a.colsOut = (a.colsIn - 3) / s + 1;
  // As many output rows as threads allow and kMaxRows input rows cover.
  a.rowsOut = kThreads / (a.colsOut * a.vecs);
  const uint32_t maxRows = (kMaxRows - 3) / s + 1;
  if (a.rowsOut > maxRows)
    a.rowsOut = maxRows;
  if (a.rowsOut > d.outH)
    a.rowsOut = d.outH;
  a.rowsIn = (a.rowsOut - 1) * s + 3;
  a.colBlocks = (d.outW + a.colsOut - 1) / a.colsOut;
  a.rowBlocks = (d.outH + a.rowsOut - 1) / a.rowsOut;
  return true;
}

} // namespace

bool depthwise3x3Takes(const DepthwiseDesc &d, int inType) {
  if (inType != kHalf || d.channels % 8 != 0 || d.kH != 3 || d.kW != 3 ||
      d.dilH != 1 || d.dilW != 1 || d.strideH != d.strideW ||
      (d.strideH != 1 && d.strideH != 2))
    return false;
  Dw3x3Args a;
  if (!shapeFor(d, a))
    return false;
  const uint64_t inBytes = uint64_t(d.batch) * d.inH * d.inW * d.channels * 2;
  const uint64_t blocks = uint64_t(d.batch) * a.rowBlocks * a.colBlocks;
  return inBytes < kOutOfRange && blocks < 0x7fffffffull;
}

hipError_t launchDepthwise3x3(const DepthwiseDesc &d, int inType,
                                 int outType, const void *in,
                                 const void *weightsPacked, const void *bias,
                                 void *out, hipStream_t stream) {
  if (!depthwise3x3Takes(d, inType))
    return hipErrorInvalidValue;
  if (uint64_t(d.batch) * d.outH * d.outW == 0)
    return hipSuccess;
  Dw3x3Args a;
  a.d = d;
  shapeFor(d, a);
  a.inBytes = uint32_t(uint64_t(d.batch) * d.inH * d.inW * d.channels * 2);
  a.divVecs = makeFastDiv(a.vecs);
  a.divColBlocks = makeFastDiv(a.colBlocks);
  a.divRowBlocks = makeFastDiv(a.rowBlocks);
  a.divOutItems = makeFastDiv(a.colsOut * a.vecs);
  const bool s1 = d.strideH == 1;
  if (outType == kHalf)
    return s1 ? run<1, __half>(a, in, weightsPacked, bias, out, stream)
              : run<2, __half>(a, in, weightsPacked, bias, out, stream);
  if (outType == kFloat)
    return s1 ? run<1, float>(a, in, weightsPacked, bias, out, stream)
              : run<2, float>(a, in, weightsPacked, bias, out, stream);
  return hipErrorInvalidValue;
}

} // namespace mxk

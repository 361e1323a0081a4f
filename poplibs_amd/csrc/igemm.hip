// Implicit-GEMM forward convolution on the CDNA4 matrix cores.
//
// GEMM view of one convolution group:
//   M = batch * outH * outW   output pixels (rows)
//   N = out channels          (columns)
//   K = kH * kW * in channels, k = (kh * kW + kw) * Ci + ci
//   A[m][k] = in[b][oh*sH + kh*dH - padH][ow*sW + kw*dW - padW][g*Ci + ci]
//             (zero outside the valid input window: padding is never stored)
//   B[k][n] = packed weights [g][n][k]  (K contiguous, zero padded)
// Both operands are therefore contiguous along K in memory, which is how an
// MFMA lane wants them: 16 bytes = 8 halves (or 16 fp8) of consecutive k.
//
// Workgroup: 256 threads = 4 wave64, tile 128 (M) x BN (N), BN = 64 or 128,
// K step of 64 bytes per row (32 halves / 64 fp8).  Each k-step the
// workgroup gathers the im2col A tile and the B tile with 16-byte global
// loads (coalesced along channels, NHWC), stages them in LDS (double
// buffered, rows padded from 64 to 80 bytes so that the 16 lanes of one LDS
// read phase hit 64 distinct banks), and each wave multiplies its 64 x BN/2
// sub-tile with v_mfma_f32_32x32x16_f16 (fp16) or
// v_mfma_f32_32x32x64_f8f6f4 (fp8), accumulating in fp32.  The next k-step's
// global loads are issued before the current step's MFMAs so that HBM/L2
// latency hides behind the matrix cores.
//
// This takes the role of PopLibs' AMP vertices ConvPartial1x1Out /
// ConvPartialnx1 (lib/poplin/codelets/ConvPartial1x1Out.cpp:49-173,
// ConvPartialnx1.cpp:52-246), including the quarter (fp8) case whose scale
// 2^(sIn + sW) is applied once to the fp32 sum
// (lib/poplin/codelets/inlineAssemblerConv.hpp:28-33).
#include "device_types.hpp"
#include "kernels.hpp"

namespace mxk {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx8 __attribute__((ext_vector_type(8)));

constexpr int kBlockM = 128;
constexpr int kRowBytes = 64;  // bytes of K per tile row and k-step
constexpr int kLdsRow = 80;    // padded LDS row pitch
constexpr int kThreads = 256;

struct IgemmArgs {
  IgemmDesc d;
  uint32_t M;        // batch * outH * outW
  uint32_t mTiles, nTiles;
  uint32_t kSteps;   // kPadded / elements per k-step
  uint32_t kPadded;  // row length of the packed weights, in elements
  uint32_t coPadded; // rows per group of the packed weights
};

/// Workgroups are dealt round-robin over the 8 XCDs, each with its own L2.
/// Give every XCD one contiguous run of tiles so that neighbouring tiles,
/// which share input halo rows and the weight tile, meet in the same L2.
__device__ __forceinline__ uint32_t xcdSwizzle(uint32_t bid, uint32_t total) {
  const uint32_t xcd = bid & 7u, idx = bid >> 3;
  const uint32_t q = total >> 3, rem = total & 7u;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

template <int EB> struct Mma;

/// fp16: two K=16 steps per 64-byte row.
template <> struct Mma<2> {
  template <int TN, int FA, int FB>
  static __device__ __forceinline__ void
  step(const char *ldsA, const char *ldsB, int lane, floatx16 (&acc)[2][TN]) {
    const int row = lane & 31, kb = (lane >> 5) * 16;
#pragma unroll
    for (int s = 0; s != 2; ++s) {
      half8 a[2], b[TN];
#pragma unroll
      for (int i = 0; i != 2; ++i)
        a[i] = *reinterpret_cast<const half8 *>(ldsA + (i * 32 + row) * kLdsRow +
                                                s * 32 + kb);
#pragma unroll
      for (int j = 0; j != TN; ++j)
        b[j] = *reinterpret_cast<const half8 *>(ldsB + (j * 32 + row) * kLdsRow +
                                                s * 32 + kb);
#pragma unroll
      for (int i = 0; i != 2; ++i)
#pragma unroll
        for (int j = 0; j != TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j],
                                                             acc[i][j], 0, 0, 0);
    }
  }
};

/// fp8: one K=64 step per 64-byte row.  FA / FB: 0 = E4M3, 1 = E5M2 (the
/// cbsz / blgp operand-format fields of the instruction).
template <> struct Mma<1> {
  template <int TN, int FA, int FB>
  static __device__ __forceinline__ void
  step(const char *ldsA, const char *ldsB, int lane, floatx16 (&acc)[2][TN]) {
    const int row = lane & 31, kb = (lane >> 5) * 32;
    // 32 bytes per lane, fetched as two 16-byte LDS reads (rows are only
    // 16-byte aligned).
    auto load32 = [](const char *p) {
      const uint4 lo = *reinterpret_cast<const uint4 *>(p);
      const uint4 hi = *reinterpret_cast<const uint4 *>(p + 16);
      return intx8{int(lo.x), int(lo.y), int(lo.z), int(lo.w),
                   int(hi.x), int(hi.y), int(hi.z), int(hi.w)};
    };
    intx8 a[2], b[TN];
#pragma unroll
    for (int i = 0; i != 2; ++i)
      a[i] = load32(ldsA + (i * 32 + row) * kLdsRow + kb);
#pragma unroll
    for (int j = 0; j != TN; ++j)
      b[j] = load32(ldsB + (j * 32 + row) * kLdsRow + kb);
#pragma unroll
    for (int i = 0; i != 2; ++i)
#pragma unroll
      for (int j = 0; j != TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
            a[i], b[j], acc[i][j], FA, FB, 0, 0, 0, 0);
  }
};

template <int BN, int EB, int FA, int FB, class OutT>
__global__ __launch_bounds__(kThreads) void igemmKernel(
    IgemmArgs a, const char *__restrict__ in, const char *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out, float scale) {
  constexpr int TN = BN / 64;              // 32-column MFMA tiles per wave
  constexpr int CE = 16 / EB;              // elements per 16-byte chunk
  constexpr int BKE = kRowBytes / EB;      // elements per k-step
  constexpr int BROWS = BN / 64;           // B rows loaded per thread
  constexpr int kTileBytes = (kBlockM + BN) * kLdsRow;
  __shared__ __align__(16) char lds[2 * kTileBytes];

  const IgemmDesc &d = a.d;
  const uint32_t tile = xcdSwizzle(blockIdx.x, gridDim.x);
  const uint32_t nTile = tile % a.nTiles;
  const uint32_t mTile = (tile / a.nTiles) % a.mTiles;
  const uint32_t g = tile / (a.nTiles * a.mTiles);

  const int t = threadIdx.x;
  const int chunk = t & 3, rowBase = t >> 2;
  const uint32_t inChans = d.groups * d.inChansPerGroup;
  const uint32_t outChans = d.groups * d.outChansPerGroup;

  // The two A rows (output pixels) this thread gathers.
  const char *rowPtr[2];
  int ihBase[2], iwBase[2];
  bool rowValid[2];
#pragma unroll
  for (int r = 0; r != 2; ++r) {
    const uint32_t m = mTile * kBlockM + rowBase + r * 64;
    rowValid[r] = m < a.M;
    const uint32_t mm = rowValid[r] ? m : 0;
    const uint32_t ow = mm % d.outW;
    const uint32_t oh = (mm / d.outW) % d.outH;
    const uint32_t b = mm / (d.outW * d.outH);
    ihBase[r] = int(oh * d.strideH) - d.padH;
    iwBase[r] = int(ow * d.strideW) - d.padW;
    rowPtr[r] = in + (size_t(b) * d.inH * d.inW * inChans +
                      size_t(g) * d.inChansPerGroup) *
                         EB;
  }
  // Position of this thread's chunk inside K, kept as (kh, kw, ci).
  uint32_t ci = chunk * CE, kw = 0, kh = 0;
  auto normalise = [&] {
    while (ci >= d.inChansPerGroup) {
      ci -= d.inChansPerGroup;
      if (++kw == d.kW) {
        kw = 0;
        ++kh;
      }
    }
  };
  normalise();

  const char *bPtr = w + ((size_t(g) * a.coPadded + nTile * BN + rowBase) *
                              a.kPadded +
                          chunk * CE) *
                             EB;
  const size_t bRowSkip = size_t(64) * a.kPadded * EB;

  uint4 aReg[2], bReg[BROWS];
  auto loadGlobal = [&] {
    const int ih0 = int(kh * d.dilH), iw0 = int(kw * d.dilW);
#pragma unroll
    for (int r = 0; r != 2; ++r) {
      const int ih = ihBase[r] + ih0, iw = iwBase[r] + iw0;
      const bool ok = rowValid[r] && kh < d.kH && ih >= int(d.loH) &&
                      ih < int(d.hiH) && iw >= int(d.loW) && iw < int(d.hiW);
      aReg[r] = ok ? *reinterpret_cast<const uint4 *>(
                         rowPtr[r] +
                         (size_t(uint32_t(ih) * d.inW + uint32_t(iw)) * inChans +
                          ci) *
                             EB)
                   : uint4{0, 0, 0, 0};
    }
#pragma unroll
    for (int r = 0; r != BROWS; ++r)
      bReg[r] = *reinterpret_cast<const uint4 *>(bPtr + r * bRowSkip);
  };
  auto storeLds = [&](int buf) {
    char *base = lds + buf * kTileBytes + rowBase * kLdsRow + chunk * 16;
#pragma unroll
    for (int r = 0; r != 2; ++r)
      *reinterpret_cast<uint4 *>(base + r * 64 * kLdsRow) = aReg[r];
#pragma unroll
    for (int r = 0; r != BROWS; ++r)
      *reinterpret_cast<uint4 *>(base + (kBlockM + r * 64) * kLdsRow) = bReg[r];
  };
  auto advance = [&] {
    ci += BKE;
    normalise();
    bPtr += kRowBytes;
  };

  const int wave = t >> 6, lane = t & 63;
  const int wm = wave >> 1, wn = wave & 1;
  floatx16 acc[2][TN];
#pragma unroll
  for (int i = 0; i != 2; ++i)
#pragma unroll
    for (int j = 0; j != TN; ++j)
#pragma unroll
      for (int v = 0; v != 16; ++v)
        acc[i][j][v] = 0.0f;

  loadGlobal();
  storeLds(0);
  __syncthreads();
  for (uint32_t kt = 0; kt != a.kSteps; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 != a.kSteps;
    if (more) {
      advance();
      loadGlobal();
    }
    const char *ldsA = lds + buf * kTileBytes + wm * 64 * kLdsRow;
    const char *ldsB =
        lds + buf * kTileBytes + (kBlockM + wn * (BN / 2)) * kLdsRow;
    Mma<EB>::template step<TN, FA, FB>(ldsA, ldsB, lane, acc);
    if (more)
      storeLds(buf ^ 1);
    __syncthreads();
  }

  // Epilogue.  Lane l of a 32x32 accumulator holds column l % 32 and rows
  // 8 * (v / 4) + 4 * (l / 32) + v % 4 for v = 0..15.
  const uint32_t col = lane & 31, rowOff = (lane >> 5) * 4;
#pragma unroll
  for (int j = 0; j != TN; ++j) {
    const uint32_t n = nTile * BN + wn * (BN / 2) + j * 32 + col;
    if (n >= d.outChansPerGroup)
      continue;
    const uint32_t c = g * d.outChansPerGroup + n;
    const float bv = bias ? Load<OutT>::at(bias, c, 0) : 0.0f;
#pragma unroll
    for (int i = 0; i != 2; ++i)
#pragma unroll
      for (int v = 0; v != 16; ++v) {
        const uint32_t m = mTile * kBlockM + wm * 64 + i * 32 + 8 * (v / 4) +
                           rowOff + (v % 4);
        if (m < a.M)
          storeOut(out, size_t(m) * outChans + c, acc[i][j][v] * scale + bv);
      }
  }
}

template <int BN, int EB, int FA, int FB, class OutT>
hipError_t run(const IgemmArgs &a, const void *in, const void *w,
               const void *bias, void *out, float scale, hipStream_t stream) {
  const uint64_t blocks = uint64_t(a.mTiles) * a.nTiles * a.d.groups;
  if (blocks == 0)
    return hipSuccess;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((igemmKernel<BN, EB, FA, FB, OutT>), dim3(uint32_t(blocks)),
                     dim3(kThreads), 0, stream, a,
                     static_cast<const char *>(in), static_cast<const char *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out),
                     scale);
  return hipGetLastError();
}

template <int BN, int EB, int FA, int FB>
hipError_t runOut(const IgemmArgs &a, int outType, const void *in,
                  const void *w, const void *bias, void *out, float scale,
                  hipStream_t stream) {
  if (outType == kHalf)
    return run<BN, EB, FA, FB, __half>(a, in, w, bias, out, scale, stream);
  if (outType == kFloat)
    return run<BN, EB, FA, FB, float>(a, in, w, bias, out, scale, stream);
  return hipErrorInvalidValue;
}

template <int BN>
hipError_t runType(const IgemmArgs &a, int inType, int outType, const void *in,
                   const void *w, const void *bias, void *out,
                   const QuarterInfo &q, hipStream_t stream) {
  if (inType == kHalf)
    return runOut<BN, 2, 0, 0>(a, outType, in, w, bias, out, 1.0f, stream);
  if (inType != kQuarter)
    return hipErrorInvalidValue;
  // Instruction format codes: 0 = E4M3, 1 = E5M2.
  const int fa = q.inFormat == kE4M3 ? 0 : 1;
  const int fb = q.weightFormat == kE4M3 ? 0 : 1;
  if (fa == 0 && fb == 0)
    return runOut<BN, 1, 0, 0>(a, outType, in, w, bias, out, q.scale, stream);
  if (fa == 0 && fb == 1)
    return runOut<BN, 1, 0, 1>(a, outType, in, w, bias, out, q.scale, stream);
  if (fa == 1 && fb == 0)
    return runOut<BN, 1, 1, 0>(a, outType, in, w, bias, out, q.scale, stream);
  return runOut<BN, 1, 1, 1>(a, outType, in, w, bias, out, q.scale, stream);
}

} // namespace

hipError_t launchIgemm(const IgemmDesc &d, int inType, int outType,
                       const void *in, const void *weightsPacked,
                       const void *bias, void *out, const QuarterInfo &q,
                       hipStream_t stream) {
  const uint32_t eb = inType == kHalf ? 2 : 1;
  const uint32_t bke = kRowBytes / eb;
  // The shapes the kernel is compiled for; the planner only produces these.
  if (d.blockM != kBlockM || (d.blockN != 64 && d.blockN != 128) ||
      d.blockK != bke || d.inChansPerGroup % (16 / eb) != 0 ||
      (inType != kHalf && inType != kQuarter))
    return hipErrorInvalidValue;
  IgemmArgs a;
  a.d = d;
  const uint64_t m = uint64_t(d.batch) * d.outH * d.outW;
  if (m > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  a.M = uint32_t(m);
  a.mTiles = (a.M + kBlockM - 1) / kBlockM;
  a.nTiles = (d.outChansPerGroup + d.blockN - 1) / d.blockN;
  a.coPadded = a.nTiles * d.blockN;
  const uint32_t k = d.kH * d.kW * d.inChansPerGroup;
  a.kPadded = (k + bke - 1) / bke * bke;
  a.kSteps = a.kPadded / bke;
  if (d.blockN == 128)
    return runType<128>(a, inType, outType, in, weightsPacked, bias, out, q,
                        stream);
  return runType<64>(a, inType, outType, in, weightsPacked, bias, out, q,
                     stream);
}

} // namespace mxk

// Pieces shared by the implicit-GEMM kernels: tile constants, the LDS tile
// layout and MFMA operand ("fragment") access, direct-to-LDS loads, the
// fence-free workgroup barrier and the epilogue that writes a finished tile.
#ifndef poplibs_amd_igemm_common_hpp
#define poplibs_amd_igemm_common_hpp
#include "device_types.hpp"
#include "kernels.hpp"

#include <type_traits>

namespace mxk {

struct IgemmArgs {
  IgemmDesc d;
  FastDiv divOutW, divOutH;
  FastDiv divInDilH, divInDilW;
  FastDiv divCiBytes, divKW; // by bytes of K per tap; by kernel width
  FastDiv divNTiles, divMTiles, divGroups; // workgroup number -> tile
  FastDiv divOutD, divKH;
  uint32_t tapRowStarts; // tap mask mode: bit kh * kW for every kernel row
  uint32_t tapPlaneStarts; // ... and bit kd * kH * kW for every kernel plane
  uint32_t outMapped; // outputs go to every outStep-th pixel of a larger field
  uint32_t outTransposed; // the final result as [channel][pixel]
  uint32_t mode;     // kMaskTaps, kRangeTaps or kDilatedTaps
  uint32_t M;        // batch * outH * outW
  uint32_t mTiles, nTiles;
  uint32_t kSteps;   // k-steps each workgroup runs (one part of K)
  uint32_t kPadded;  // row length of the packed weights, in elements
  uint32_t coPadded; // rows per group of the packed weights
  uint64_t inBytes;    // size of the input tensor
  uint32_t imageBytes; // ... and of one image (batch element) of it
  uint32_t wBytes;   // size of the packed weights
};

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

/// Compile-time loop: body(std::integral_constant<int, I>) for I in [0, N).
template <int I, int N, class F>
__device__ __forceinline__ void staticFor(F &&body) {
  if constexpr (I < N) {
    body(std::integral_constant<int, I>{});
    staticFor<I + 1, N>(body);
  }
}

constexpr int kBlockM = 128;
constexpr int kRowBytes = 128; // bytes of K per tile row and k-step
constexpr int kThreads = 512;  // 4 consumer + 4 producer waves
constexpr int kProducers = 256; // threads that move data
constexpr int kChunks = kRowBytes / 16; // 16-byte chunks per row
constexpr int kRowsPerPass = kProducers / kChunks; // rows per producer pass
constexpr int kLoadBytes = 64 * 16; // LDS bytes one wave-wide load fills
constexpr uint32_t kOutOfRange = 0x80000000u; // beyond any buffer we accept


/// Workgroups are dealt round-robin over the 8 XCDs, each with its own L2.
/// Give every XCD one contiguous run of tiles so that neighbouring tiles,
/// which share input halo rows and the weight tile, meet in the same L2.
__device__ __forceinline__ uint32_t xcdSwizzle(uint32_t bid, uint32_t total) {
  const uint32_t xcd = bid & 7u, idx = bid >> 3;
  const uint32_t q = total >> 3, rem = total & 7u;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t bufferOf(const void *p,
                                                           uint32_t bytes) {
  // Raw (stride 0) buffer of `bytes` bytes; 32-bit data format.
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), short(0),
                                           int(bytes), 0x00020000);
}

/// `wait until at most n vector-memory operations are outstanding`, leaving
/// the other counters alone (gfx9 encoding of s_waitcnt).
#define MXK_WAIT_VMCNT(n)                                                      \
  __builtin_amdgcn_s_waitcnt(((n)&15) | (((n) >> 4) << 14) | (7 << 4) |       \
                             (15 << 8))

/// Wait for this wave's LDS reads (and scalar loads) only.
#define MXK_WAIT_LGKMCNT0() __builtin_amdgcn_s_waitcnt(0xC07F)

/// Workgroup barrier without the release / acquire fences of
/// __syncthreads().  Those fences would drain every outstanding buffer load
/// (a load that writes LDS counts as a pending LDS write) at each k-step and
/// with it the whole prefetch queue.  The callers wait for exactly what the
/// other side needs - producers: the oldest stage's loads; consumers: their
/// own LDS reads - before arriving here.
__device__ __forceinline__ void stepBarrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

using LdsPtr = __attribute__((address_space(3))) void *;

/// 16 bytes per lane from a buffer straight into LDS: lane l's data lands at
/// dst + 16 l (dst is wave-uniform).  Out-of-range offsets deliver zeros.
/// The builtin exists for the GPU target only; the host compilation pass,
/// which merely needs the kernels' launch stubs, sees an empty body.
/// POLICY: the load's cache policy bits - 0, or kStreamingLoad for data that
/// is read once.
constexpr int kStreamingLoad = 2;
/// Cache policy of a store that goes through the L2 to memory at once
/// (device scope) instead of leaving a dirty line there.  What a kernel leaves
/// dirty in the eight L2s is written back when it ends, before the next kernel
/// of the stream starts; for a kernel of a few microseconds whose output comes
/// all at its end that write-back is a measurable part (3x3 on 28x28, 128
/// channels: 9.1 -> 8.9 us).  Kernels that stream their output while they run
/// lose by it (1x1 on 56x56: 12.3 -> 15.5 us).
constexpr int kWriteThroughStore = 16;
template <int POLICY = 0>
__device__ __forceinline__ void loadToLds(__amdgpu_buffer_rsrc_t buffer,
                                          LdsPtr dst, uint32_t vectorOffset,
                                          uint32_t scalarOffset) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(buffer, dst, 16, vectorOffset,
                                           scalarOffset, 0, POLICY);
#endif
}

template <int EB> struct Mma;

/// Where a lane finds its MFMA operands in LDS.  Rows are split into 16-byte
/// chunks; chunk c of a row sits at chunk position c ^ swizzle of that row.
/// a[i]: byte address of the lane's row of the i-th 32-row block of the A
/// operand, with its swizzle; chunkBase: first chunk of the k-step inside
/// that row (0 when a row holds just the k-step).  b: the lane's row of the
/// first 32-row block of the B tile; further blocks follow at 32 tile rows.
struct FragmentAddress {
  const char *a[2];
  int swizzleA[2];
  int chunkBase;
  const char *b;
  int swizzleB;
};

/// Tile rows in LDS are 128 bytes.  Row r sits at row position
/// r ^ ((r >> 3) & 1), its chunk c at chunk position c ^ (r & 7).  A wave reads
/// fragments of 32-row blocks whose bases are multiples of 32, so both depend
/// on the lane only: this is the byte offset of (row lane & 31, chunk 0)
/// before the chunk XOR.
__device__ __forceinline__ int fragmentRowOffset(int lane) {
  return ((lane & 31) ^ ((lane >> 3) & 1)) * kRowBytes;
}

/// The MFMA operands ("fragments") of one consumer wave.  A k-step is split
/// into kSubSteps sub-steps; fragment set s holds what sub-step s multiplies.
/// load<S> issues the LDS reads of one set, mul<S> the MFMAs that consume it:
/// the first MFMA, then `between()` (the caller's LDS reads for a later
/// sub-step, so that they are in flight under the remaining MFMAs), then the
/// rest.  The weights are the MFMA's row operand, so an accumulator holds the
/// transposed block: lane = output pixel, registers = output channels.

/// fp16: 4 sub-steps of K=16, 32 bytes (two chunks, one per half-wave) each.
template <> struct Mma<2> {
  static constexpr int kSubSteps = kRowBytes / 32;
  template <int TN> struct Frags {
    half8 a[kSubSteps][2], b[kSubSteps][TN];
  };
  template <int S, int TN>
  static __device__ __forceinline__ void load(const FragmentAddress &at,
                                              int lane, Frags<TN> &f) {
    const int c = S * 2 + (lane >> 5);
#pragma unroll
    for (int i = 0; i != 2; ++i)
      f.a[S][i] = *reinterpret_cast<const half8 *>(
          at.a[i] + (((at.chunkBase + c) ^ at.swizzleA[i]) << 4));
#pragma unroll
    for (int j = 0; j != TN; ++j)
      f.b[S][j] = *reinterpret_cast<const half8 *>(
          at.b + j * 32 * kRowBytes + ((c ^ at.swizzleB) << 4));
  }
  template <int S, int TN, int FA, int FB, class F>
  static __device__ __forceinline__ void
  mul(const Frags<TN> &f, floatx16 (&acc)[2][TN], F &&between) {
#pragma unroll
    for (int i = 0; i != 2; ++i)
#pragma unroll
      for (int j = 0; j != TN; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
            f.b[S][j], f.a[S][i], acc[i][j], 0, 0, 0);
        if (i == 0 && j == 0)
          between();
      }
  }
};

/// fp32: 4 sub-steps of 8 values, 32 bytes (two chunks, one per half-wave)
/// each.  The fp32 MFMA takes one value per lane (K = 2: one from either
/// half-wave), so the four values of a lane's chunk feed four MFMAs; which
/// k meets which is the same for both operands, and that is all that counts.
template <> struct Mma<4> {
  static constexpr int kSubSteps = kRowBytes / 32;
  template <int TN> struct Frags {
    floatx4 a[kSubSteps][2], b[kSubSteps][TN];
  };
  template <int S, int TN>
  static __device__ __forceinline__ void load(const FragmentAddress &at,
                                              int lane, Frags<TN> &f) {
    const int c = S * 2 + (lane >> 5);
#pragma unroll
    for (int i = 0; i != 2; ++i)
      f.a[S][i] = *reinterpret_cast<const floatx4 *>(
          at.a[i] + (((at.chunkBase + c) ^ at.swizzleA[i]) << 4));
#pragma unroll
    for (int j = 0; j != TN; ++j)
      f.b[S][j] = *reinterpret_cast<const floatx4 *>(
          at.b + j * 32 * kRowBytes + ((c ^ at.swizzleB) << 4));
  }
  template <int S, int TN, int FA, int FB, class F>
  static __device__ __forceinline__ void
  mul(const Frags<TN> &f, floatx16 (&acc)[2][TN], F &&between) {
    // the four MFMAs into one accumulator depend on each other: the other
    // accumulators' go in between
#pragma unroll
    for (int e = 0; e != 4; ++e)
#pragma unroll
      for (int i = 0; i != 2; ++i)
#pragma unroll
        for (int j = 0; j != TN; ++j) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              f.b[S][j][e], f.a[S][i][e], acc[i][j], 0, 0, 0);
          if (e == 0 && i == 0 && j == 0)
            between();
        }
  }
};

/// fp8: 2 sub-steps of K=64, 64 bytes (four chunks, two per half-wave) each.
/// FA / FB: 0 = E4M3, 1 = E5M2 (the cbsz / blgp operand-format fields).
template <> struct Mma<1> {
  static constexpr int kSubSteps = kRowBytes / 64;
  template <int TN> struct Frags {
    intx8 a[kSubSteps][2], b[kSubSteps][TN];
  };
  template <int S, int TN>
  static __device__ __forceinline__ void load(const FragmentAddress &at,
                                              int lane, Frags<TN> &f) {
    const int c0 = S * 4 + (lane >> 5) * 2;
    // 32 bytes per lane: two chunks that the swizzle may have separated.
    auto load32 = [&](const char *row, int chunk, int swizzle) {
      const uintx4 lo =
          *reinterpret_cast<const uintx4 *>(row + ((chunk ^ swizzle) << 4));
      const uintx4 hi = *reinterpret_cast<const uintx4 *>(
          row + (((chunk + 1) ^ swizzle) << 4));
      return intx8{int(lo.x), int(lo.y), int(lo.z), int(lo.w),
                   int(hi.x), int(hi.y), int(hi.z), int(hi.w)};
    };
#pragma unroll
    for (int i = 0; i != 2; ++i)
      f.a[S][i] = load32(at.a[i], at.chunkBase + c0, at.swizzleA[i]);
#pragma unroll
    for (int j = 0; j != TN; ++j)
      f.b[S][j] = load32(at.b + j * 32 * kRowBytes, c0, at.swizzleB);
  }
  template <int S, int TN, int FA, int FB, class F>
  static __device__ __forceinline__ void
  mul(const Frags<TN> &f, floatx16 (&acc)[2][TN], F &&between) {
#pragma unroll
    for (int i = 0; i != 2; ++i)
#pragma unroll
      for (int j = 0; j != TN; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
            f.b[S][j], f.a[S][i], acc[i][j], FB, FA, 0, 0, 0, 0);
        if (i == 0 && j == 0)
          between();
      }
  }
};

/// LDS bytes the epilogue needs for a 128 x BN tile of OutT.
template <int BN, class OutT> constexpr int epilogueLdsBytes() {
  return kBlockM * (BN * int(sizeof(OutT)) + 16);
}

/// LDS of a workgroup: the stages and the row table - or the output tile, if
/// that is larger (two stages and fp32 outputs).
template <int BN, int NS, class OutT> constexpr int igemmLdsBytes() {
  constexpr int loop =
      NS * (kBlockM + BN) * kRowBytes +
      kBlockM * int(sizeof(uint2) + sizeof(uint32_t));
  return loop > epilogueLdsBytes<BN, OutT>() ? loop
                                             : epilogueLdsBytes<BN, OutT>();
}

/// Writes the workgroup's finished 128 x BN tile.  Call with every wave past
/// its last use of LDS (a workgroup barrier behind it): LDS is reused from
/// offset 0.
template <int BN, class OutT>
__device__ __forceinline__ void
igemmEpilogue(char *lds, const IgemmArgs &a, floatx16 (&acc)[2][BN / 64],
              bool producer, int t, int lane, int wm, int wn, uint32_t mTile,
              uint32_t nTile, uint32_t g, const OutT *__restrict__ bias,
              OutT *__restrict__ out, float scale) {
  constexpr int TN = BN / 64;
  const IgemmDesc &d = a.d;
  const uint32_t outChans = d.groups * d.outChansPerGroup;
  // Epilogue.  All k-steps are consumed and every wave is past the last
  // barrier, so LDS is free: the consumers lay the finished tile out as
  // [128 rows][BN outputs] (+ 16 bytes of padding per row), then everybody
  // copies it out.  The weights were the MFMA's row operand, so lane l of a
  // 32x32 accumulator holds output pixel l % 32 and output channels
  // 8 * (v / 4) + 4 * (l / 32) + v % 4 for v = 0..15: runs of four channels,
  // contiguous in the channels-last output, that go to LDS as one vector.
  constexpr int kOutRow = BN * int(sizeof(OutT)) + 16;
  if (!producer) {
    const uint32_t mRow = lane & 31, nOff4 = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j != TN; ++j)
#pragma unroll
      for (int q = 0; q != 4; ++q) {
        const uint32_t nLocal = wn * (BN / 2) + j * 32 + 8 * q + nOff4;
        float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (bias) {
          const uint32_t n = nTile * BN + nLocal;
#pragma unroll
          for (int e = 0; e != 4; ++e)
            if (n + e < d.outChansPerGroup)
              bv[e] = Load<OutT>::at(bias, g * d.outChansPerGroup + n + e, 0);
        }
#pragma unroll
        for (int i = 0; i != 2; ++i) {
          const uint32_t mLocal = wm * 64 + i * 32 + mRow;
          float v[4];
#pragma unroll
          for (int e = 0; e != 4; ++e)
            v[e] = acc[i][j][q * 4 + e] * scale + bv[e];
          storeOut4(reinterpret_cast<OutT *>(lds + mLocal * kOutRow) + nLocal,
                    v);
        }
      }
  }
  __syncthreads();
  constexpr int kVecElems = 16 / int(sizeof(OutT));
  constexpr int kVecsPerRow = BN / kVecElems;
  // 16-byte stores need the channel count (hence every row start) to be a
  // multiple of the vector; otherwise fall back to single elements.
  const bool vectorOk = outChans % kVecElems == 0 &&
                        d.outChansPerGroup % kVecElems == 0;
  for (int idx = t; idx < kBlockM * kVecsPerRow; idx += kThreads) {
    const uint32_t mLocal = idx / kVecsPerRow, vec = idx % kVecsPerRow;
    const uint32_t m = mTile * kBlockM + mLocal;
    const uint32_t n = nTile * BN + vec * kVecElems;
    if (m >= a.M || n >= d.outChansPerGroup)
      continue;
    const char *src = lds + mLocal * kOutRow + vec * 16;
    // the output pixel of row m: m itself, or - one phase of a convolution
    // over a zero-stuffed input - every outStep-th pixel of a larger field
    size_t pixel = m;
    if (a.outMapped) {
      const uint32_t q = a.divOutW(m), ow = m - q * d.outW;
      const uint32_t q2 = a.divOutH(q), oh = q - q2 * d.outH;
      const uint32_t image = a.divOutD(q2), od = q2 - image * d.outD;
      pixel = ((size_t(image) * d.outFullD + od * d.outStepD + d.outOffD) *
                   d.outFullH +
               oh * d.outStepH + d.outOffH) *
                  d.outFullW +
              ow * d.outStepW + d.outOffW;
    }
    if (a.outTransposed) {
      // [channel][pixel]: element stores, for small outputs
      const OutT *e = reinterpret_cast<const OutT *>(src);
      for (int k = 0; k != kVecElems && n + k < d.outChansPerGroup; ++k)
        out[size_t(g * d.outChansPerGroup + n + k) * a.M + m] = e[k];
      continue;
    }
    OutT *dst = out + pixel * outChans + g * d.outChansPerGroup + n;
    if (vectorOk) {
      *reinterpret_cast<uintx4 *>(dst) = *reinterpret_cast<const uintx4 *>(src);
    } else {
      const OutT *e = reinterpret_cast<const OutT *>(src);
      for (int k = 0; k != kVecElems && n + k < d.outChansPerGroup; ++k)
        dst[k] = e[k];
    }
  }
}

} // namespace
} // namespace mxk
#endif

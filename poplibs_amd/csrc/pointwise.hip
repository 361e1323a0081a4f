// Pointwise (1x1, stride 1, unpadded) forward convolution with few input
// channels: a tall, skinny GEMM - M = batch * H * W pixels, K = Ci, N = Co -
// that is bound by HBM, not by the matrix cores (PopLibs serves it with
// ConvPartial1x1Out, lib/poplin/codelets/ConvPartial1x1Out.cpp:49-173).
//
// igemm.hip's big tiles and deep k-pipeline have nothing to pipeline here:
// with K = 256 a 128-pixel tile is four k-steps of prologue and epilogue.
// This kernel streams instead:
//   * a workgroup is 2 to 8 compute waves + 2 or 4 loader waves and owns 64,
//     128 or 256 output channels; it walks over tiles of 32 to 128 pixels,
//     all of K each, and multiplies a tile by its channels 64 at a time;
//   * the weights never touch LDS: they are packed per (32-channel block,
//     16-deep k-slice) in MFMA operand order, each compute wave fetches its
//     block once - one coalesced 16-byte load per lane and slice - and keeps
//     it in registers for all its tiles.  (Fetching them per tile was
//     measured to cost as much vector-cache bandwidth as the activations.)
//   * the loader wave brings the activation rows of a tile (contiguous in
//     the channels-last tensor) straight into a ring of 3 or 4 LDS buffers
//     with 1 KB direct-to-LDS loads, 2 or 3 tiles ahead of the compute waves;
//     row r's 16-byte chunk c is stored at chunk position c ^ (r & 15), so
//     that an MFMA operand read - 32 rows, one chunk - is spread over all 64
//     LDS banks (rows are a multiple of 256 bytes).  It issues nothing but
//     loads, so it can wait for exactly the oldest tile; the compute waves
//     issue nothing but stores and never wait for memory;
//   * each compute wave owns one 32 x 32 block of the tile: Ci / 16 MFMAs
//     (v_mfma_f32_32x32x16_f16, fp32 accumulate), weights as the row operand,
//     so a lane ends up with runs of 4 consecutive output channels of one
//     pixel; the block is transposed through a wave-private piece of LDS and
//     leaves as 16-byte stores, 64 bytes per pixel and store;
//   * one workgroup barrier per tile: the tile has landed / the buffer before
//     it has been read.
//
// Input channels per group: any multiple of 8 up to 512.  The kernel is
// compiled for rows of 16, 32, 64, 128, 256 and 512 channels; a layer in
// between runs as the next one up, its rows padded in LDS only - the loads of
// the 16-byte chunks past the layer's channels lie beyond the buffer and
// bring zeros without touching memory, and the packed weights carry zeros
// there.
#include "igemm_common.hpp"

namespace mxk {
namespace {

/// The row the kernel is compiled for: the next of 16, 32, ..., 512 channels.
constexpr uint32_t pwPaddedChans(uint32_t ci) {
  uint32_t p = 16;
  while (p < ci)
    p *= 2;
  return p;
}

/// A layer's input channels per group in units of two bytes - fp16 channels,
/// or pairs of fp8 ones: rows, tiles and rings are a matter of bytes.
constexpr uint32_t pwRowChans(const PointwiseDesc &d) {
  return d.inChansPerGroup * d.elemBytes / 2;
}

constexpr int kPwChans = 64;         // output channels per workgroup
constexpr int kPwStageRow = 64 + 16; // staging: 64 bytes of a pixel + padding
constexpr int kPwPairRow = 128 + 16; // ... 128 bytes: two blocks' channels

struct PwArgs {
  PointwiseDesc d;
  uint32_t M;          // batch * pixels per image
  uint32_t mTiles, nTiles;
  uint32_t nBlocks;    // 32-channel blocks per group in the packed weights
  uint32_t walkers;    // workgroups sharing the pixel tiles of one (g, nTile)
  uint32_t inBytes, wBytes;
  // fp8: 2^(scaleIn + scaleWeights), applied to the sums on their way out,
  // and its inverse, by which the bias enters them
  float scale, invScale;
};

/// One 32-byte k-slice of a 32 x 32 block: `w` and `x` are a lane's 16 bytes
/// of the weights' and the pixels' rows.  F = 0: fp16, one MFMA of K = 16
/// (the lane's 8 halves are k = 8 (lane / 32) ...).  F > 0: fp8, activations'
/// format (F - 1) & 1 and weights' (F - 1) >> 1 (0 = E4M3, 1 = E5M2): two MFMAs
/// of K = 16 on the low and the high 8 bytes - which 16 channels of the slice
/// a lane multiplies does not matter as long as the weights are packed alike.
template <int F>
__device__ __forceinline__ floatx16 pwMma(const uintx4 &w, const uintx4 &x,
                                          floatx16 acc) {
  if constexpr (F == 0) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(half8, w), __builtin_bit_cast(half8, x), acc, 0, 0,
        0);
  } else {
    const long w0 = long(uint64_t(w.x) | (uint64_t(w.y) << 32));
    const long w1 = long(uint64_t(w.z) | (uint64_t(w.w) << 32));
    const long x0 = long(uint64_t(x.x) | (uint64_t(x.y) << 32));
    const long x1 = long(uint64_t(x.z) | (uint64_t(x.w) << 32));
    constexpr int FA = (F - 1) & 1, FB = (F - 1) >> 1;
    if constexpr (FB == 0 && FA == 0) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(w0, x0, acc, 0, 0, 0);
      return __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(w1, x1, acc, 0, 0, 0);
    } else if constexpr (FB == 0 && FA == 1) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_bf8(w0, x0, acc, 0, 0, 0);
      return __builtin_amdgcn_mfma_f32_32x32x16_fp8_bf8(w1, x1, acc, 0, 0, 0);
    } else if constexpr (FB == 1 && FA == 0) {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf8_fp8(w0, x0, acc, 0, 0, 0);
      return __builtin_amdgcn_mfma_f32_32x32x16_bf8_fp8(w1, x1, acc, 0, 0, 0);
    } else {
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(w0, x0, acc, 0, 0, 0);
      return __builtin_amdgcn_mfma_f32_32x32x16_bf8_bf8(w1, x1, acc, 0, 0, 0);
    }
  }
}

/// KS: k-slices of 16 channels (Ci / 16).  TM: pixels per tile (32, 64, 128);
/// the workgroup has TM / 16 compute waves and LW loader waves, which take
/// the loads of a tile in turn.  NB: tile buffers in LDS; NB - 1 tiles are in
/// flight.  NT: 64-channel tiles of the output a workgroup owns (a.nTiles
/// counts the workgroups' shares, NT * 64 channels each): a layer that widens
/// the channels reads its input once per share, so fewer, wider shares read
/// less - 64 -> 256 channels on N = 32, 56 x 56: four shares of 64 re-read
/// 13 MB four times beside 51 MB of output.
/// F: the operands' type, see pwMma (a k-slice is 32 bytes of a row: 16 fp16
/// channels or 32 fp8 ones).
template <int KS, int TM, int NB, int LW, int NT, class OutT, int F = 0>
__global__ __launch_bounds__(TM * 4 + 64 * LW) void pointwiseKernel(
    PwArgs a, const char *__restrict__ in, const char *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out) {
  constexpr int kRow = KS * 32;                 // bytes of one activation row
  constexpr int kChunkBits = KS == 1   ? 1
                             : KS == 2 ? 2
                             : KS == 4 ? 3
                             : KS == 8 ? 4
                             : KS == 16 ? 5
                                        : 6; // log2(kRow / 16)
  // chunk c of row r sits at chunk position c ^ (r & kSwizzle)
  constexpr uint32_t kSwizzle = KS == 1 ? 1u : KS == 2 ? 3u : KS == 4 ? 7u : 15u;
  constexpr int kRowsPerLoad = 1024 / kRow;
  constexpr int kLoads = TM / kRowsPerLoad; // wave-wide loads per tile
  constexpr int kTileBytes = TM * kRow;
  constexpr int kComputeWaves = TM / 16;
  static_assert(kLoads % LW == 0, "the loader waves share a tile evenly");
  constexpr int kOwnLoads = kLoads / LW; // ... per loader wave
  static_assert((NB - 2) * kOwnLoads <= 63, "wait count fits s_waitcnt");
  // NB tile buffers | staging | bias of the workgroup's channels (fp32)
  extern __shared__ __align__(16) char lds[];

  const PointwiseDesc &d = a.d;
  // The workgroups that take the same pixel tiles for different channels
  // are neighbours in an XCD's run of workgroups: they start together and
  // meet in its L2, which then fetches a tile once for all of them.  (Dealt
  // out walker-fastest they land on different XCDs unless the walkers are a
  // multiple of eight: N = 32, 56 x 56, 128 -> 256 channels with 61 walkers
  // 25.1 us, with 56 of them 14.8.)
  const uint32_t logical =
      a.nTiles > 1 ? xcdSwizzle(blockIdx.x, gridDim.x) : blockIdx.x;
  const uint32_t nTile = logical % a.nTiles;
  const uint32_t walker = (logical / a.nTiles) % a.walkers;
  const uint32_t g = logical / (a.walkers * a.nTiles);
  const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
  const uint32_t groupBytes =
      d.inChansPerGroup * d.elemBytes; // (may be below kRow)
  const uint32_t pixelBytes = d.groups * groupBytes;

  if (wave >= kComputeWaves) {
    const int loader = wave - kComputeWaves;
    // ---- loader.  Load L of a tile fills bytes [1024 L, 1024 L + 1024) of
    // its buffer, i.e. rows L * kRowsPerLoad ...; lane l holds chunk position
    // l % (kRow / 16) of row l / (kRow / 16).
    const __amdgpu_buffer_rsrc_t inBuf = bufferOf(in, a.inBytes);
    const uint32_t rowInLoad = lane >> kChunkBits;
    const uint32_t pos = lane & ((1 << kChunkBits) - 1);
    auto issue = [&](uint32_t mTile, char *buffer) {
#pragma unroll
      for (int own = 0; own != kOwnLoads; ++own) {
        const uint32_t load = own * LW + loader;
        const uint32_t row = load * kRowsPerLoad + rowInLoad;
        const uint32_t chunk = pos ^ (row & kSwizzle);
        const uint32_t m = mTile * TM + row;
        loadToLds(inBuf, (LdsPtr)(buffer + load * 1024),
                  m < a.M && chunk * 16 < groupBytes
                      ? m * pixelBytes + g * groupBytes + chunk * 16
                      : kOutOfRange,
                  0);
      }
    };
    // Tiles this walker has no more of are "loaded" all the same, from
    // beyond the tensor (nothing is fetched): the count of loads in flight
    // stays what the waits below assume.
#pragma unroll
    for (int s = 0; s != NB - 1; ++s)
      issue(walker + s * a.walkers, lds + s * kTileBytes);
    uint32_t buffer = NB - 1; // where tile i + NB - 1 goes
    for (uint32_t mTile = walker; mTile < a.mTiles; mTile += a.walkers) {
      MXK_WAIT_VMCNT((NB - 2) * kOwnLoads);
      stepBarrier(); // tile i is in LDS; the buffer before it has been read
      issue(mTile + (NB - 1) * a.walkers, lds + buffer * kTileBytes);
      if (++buffer == NB)
        buffer = 0;
    }
    MXK_WAIT_VMCNT(0);
    return;
  }

  // ---- compute waves.  This wave's weights -> registers: block nb of the
  // two 32-channel blocks, every k-slice.
  const int mb = wave >> 1, nb = wave & 1;
  uintx4 wf[NT][KS];
#pragma unroll
  for (int nt = 0; nt != NT; ++nt) {
    const uintx4 *src =
        reinterpret_cast<const uintx4 *>(w) +
        (size_t(g * a.nBlocks + nTile * NT * 2 + nb * NT + nt) * KS) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks != KS; ++ks)
      wf[nt][ks] = src[ks * 64];
  }
  // (fp8: the sums are scaled on their way out, so the bias enters them
  // divided by the scale - a power of two)
  const float biasScale = F == 0 ? 1.0f : a.invScale;
  // One channel tile: the bias of this lane's channels 8 q + 4 (lane / 32) +
  // e stays in registers.  More: the workgroup's bias waits in LDS (registers
  // hold the weights), visible to all behind the first tile's barrier.
  float biasV[NT == 1 ? 16 : 1] = {};
  if constexpr (NT == 1) {
#pragma unroll
    for (int v = 0; v != 16; ++v) {
      const uint32_t n =
          nTile * kPwChans + nb * 32 + 8 * (v / 4) + 4 * (lane >> 5) + v % 4;
      biasV[v] = bias && n < d.outChansPerGroup
                     ? Load<OutT>::at(bias, g * d.outChansPerGroup + n, 0) *
                           biasScale
                     : 0.0f;
    }
  }
  float *biasLds = reinterpret_cast<float *>(
      lds + NB * kTileBytes + kComputeWaves * 32 * kPwStageRow);
  if (NT > 1 && bias) {
    for (uint32_t i = t; i < NT * kPwChans; i += kComputeWaves * 64) {
      const uint32_t n = nTile * NT * kPwChans + i;
      biasLds[i] = n < d.outChansPerGroup
                       ? Load<OutT>::at(bias, g * d.outChansPerGroup + n, 0) *
                             biasScale
                       : 0.0f;
    }
    MXK_WAIT_LGKMCNT0();
  }
  const uint32_t rowLocal = mb * 32 + (lane & 31);
  const uint32_t swizzle = rowLocal & kSwizzle, half = lane >> 5;
  char *stage = lds + NB * kTileBytes + wave * 32 * kPwStageRow;
  const uint32_t outChans = d.groups * d.outChansPerGroup;
  // Output leaves in passes of 64 bytes per pixel: all 32 channels of the
  // block (fp16) or 16 of them (fp32).
  constexpr int kPassChans = 64 / int(sizeof(OutT));
  constexpr int kVecElems = 16 / int(sizeof(OutT));

  uint32_t buffer = 0;
  for (uint32_t mTile = walker; mTile < a.mTiles; mTile += a.walkers) {
    stepBarrier(); // tile i has landed
    const char *rowPtr = lds + buffer * kTileBytes + rowLocal * kRow;
    if (++buffer == NB)
      buffer = 0;
    if constexpr (NT % 2 == 0 && sizeof(OutT) == 2) {
      // Two adjacent 32-channel blocks at a time: one read of the pixels
      // feeds both, and their 64 channels leave as 128 contiguous bytes per
      // pixel and store - whole lines, where a block alone writes half of
      // one.  (64 -> 256 channels on N = 32, 56 x 56: 16.1 us with one
      // 64-channel tile per workgroup, 14.5 with four and a wave's blocks
      // adjacent; storing them together or even fully contiguously changes
      // no more than 5 % of that, and neither do the staging waits: the
      // layer's 51 MB of output take 9.6 us as a plain fill.)  Sixteen pixels
      // at a time fit the wave's staging block.
      static_assert(16 * kPwPairRow <= 32 * kPwStageRow, "staging fits");
#pragma unroll
      for (int np = 0; np != NT / 2; ++np) {
        floatx16 acc[2];
#pragma unroll
        for (int j = 0; j != 2; ++j) {
          if (bias) {
            const float *b =
                biasLds + (nb * NT + 2 * np + j) * 32 + 4 * half;
#pragma unroll
            for (int q = 0; q != 4; ++q) {
              const floatx4 four =
                  *reinterpret_cast<const floatx4 *>(b + 8 * q);
#pragma unroll
              for (int e = 0; e != 4; ++e)
                acc[j][4 * q + e] = four[e];
            }
          } else {
#pragma unroll
            for (int v = 0; v != 16; ++v)
              acc[j][v] = 0.0f;
          }
        }
#pragma unroll
        for (int ks = 0; ks != KS; ++ks) {
          const uintx4 x = *reinterpret_cast<const uintx4 *>(
              rowPtr + (((ks * 2 + half) ^ swizzle) << 4));
#pragma unroll
          for (int j = 0; j != 2; ++j)
            acc[j] = pwMma<F>(wf[2 * np + j][ks], x, acc[j]);
        }
#pragma unroll
        for (int ph = 0; ph != 2; ++ph) {
          if (((lane >> 4) & 1) == ph) {
#pragma unroll
            for (int j = 0; j != 2; ++j)
#pragma unroll
              for (int q = 0; q != 4; ++q) {
                float v[4];
#pragma unroll
                for (int e = 0; e != 4; ++e)
                  v[e] = F == 0 ? acc[j][q * 4 + e]
                                : acc[j][q * 4 + e] * a.scale;
                storeOut4(
                    reinterpret_cast<OutT *>(stage + (lane & 15) * kPwPairRow) +
                        (32 * j + 8 * q + 4 * half),
                    v);
              }
          }
          MXK_WAIT_LGKMCNT0(); // (wave-private staging)
#pragma unroll
          for (int i = 0; i != 2; ++i) {
            const uint32_t u = lane + 64 * i;
            const uint32_t r = u >> 3, vec = u & 7;
            const uint32_t m = mTile * TM + mb * 32 + ph * 16 + r;
            const uint32_t n =
                nTile * NT * kPwChans + (nb * NT + 2 * np) * 32 + vec * 8;
            const uintx4 data = *reinterpret_cast<const uintx4 *>(
                stage + r * kPwPairRow + vec * 16);
            if (m < a.M && n < d.outChansPerGroup)
              __builtin_nontemporal_store(
                  data, reinterpret_cast<uintx4 *>(
                            out + size_t(m) * outChans +
                            g * d.outChansPerGroup + n));
          }
          MXK_WAIT_LGKMCNT0(); // read before the next pixels overwrite it
        }
      }
    } else
#pragma unroll
    for (int nt = 0; nt != NT; ++nt) {
      floatx16 acc;
      if constexpr (NT == 1) {
#pragma unroll
        for (int v = 0; v != 16; ++v)
          acc[v] = biasV[v];
      } else if (bias) {
        // lane's channels 8 q + 4 (lane / 32) + e of the block
        const float *b = biasLds + (nb * NT + nt) * 32 + 4 * half;
#pragma unroll
        for (int q = 0; q != 4; ++q) {
          const floatx4 four = *reinterpret_cast<const floatx4 *>(b + 8 * q);
#pragma unroll
          for (int e = 0; e != 4; ++e)
            acc[4 * q + e] = four[e];
        }
      } else {
#pragma unroll
        for (int v = 0; v != 16; ++v)
          acc[v] = 0.0f;
      }
#pragma unroll
      for (int ks = 0; ks != KS; ++ks) {
        const uintx4 x = *reinterpret_cast<const uintx4 *>(
            rowPtr + (((ks * 2 + half) ^ swizzle) << 4));
        acc = pwMma<F>(wf[nt][ks], x, acc);
      }
      // lane = pixel lane % 32, registers = channels 8 (v / 4) + 4 (lane /
      // 32) + v % 4: transpose through this wave's staging block and store.
#pragma unroll
      for (int pass = 0; pass != 32 / kPassChans; ++pass) {
#pragma unroll
        for (int q = pass * (kPassChans / 8);
             q != (pass + 1) * (kPassChans / 8); ++q) {
          float v[4];
#pragma unroll
          for (int e = 0; e != 4; ++e)
            v[e] = F == 0 ? acc[q * 4 + e] : acc[q * 4 + e] * a.scale;
          storeOut4(
              reinterpret_cast<OutT *>(stage + (lane & 31) * kPwStageRow) +
                  (8 * q + 4 * half - pass * kPassChans),
              v);
        }
        // wave-private: only this wave's LDS writes have to be visible
        MXK_WAIT_LGKMCNT0();
        const uint32_t vec = lane & 3; // 4 x 16 bytes per pixel and pass
        const uint32_t n = nTile * NT * kPwChans + (nb * NT + nt) * 32 +
                           pass * kPassChans + vec * kVecElems;
#pragma unroll
        for (int rows = 0; rows != 2; ++rows) {
          const uint32_t r = rows * 16 + (lane >> 2);
          const uint32_t m = mTile * TM + mb * 32 + r;
          const uintx4 data = *reinterpret_cast<const uintx4 *>(
              stage + r * kPwStageRow + vec * 16);
          if (m < a.M && n < d.outChansPerGroup) {
            uintx4 *dst = reinterpret_cast<uintx4 *>(
                out + size_t(m) * outChans + g * d.outChansPerGroup + n);
            // streaming store (the output is not read again here): 15.2 ->
            // 12.4 us on the 56 x 56, 256 -> 64 layer.  The same hint on the
            // loads loses a microsecond of that.
            __builtin_nontemporal_store(data, dst);
          }
        }
        MXK_WAIT_LGKMCNT0(); // staging is read before the next pass rewrites it
      }
    }
  }
}

/// Weights [G][Co][Ci] -> [G][32-channel block][k-slice][lane][16 bytes]:
/// lane l of a slice holds channel l % 32 of the block, and of its input
/// channels the E = 8 (fp16) or 16 (fp8) from 2 E slice + E (l / 32) on - the
/// row operand of pwMma.  Channels past Co are zero, and so are input channels
/// past Ci (the slices run to the padded row, `slices` of 32 bytes).
template <class T>
__global__ __launch_bounds__(256) void packPointwiseWeightsKernel(
    const T *__restrict__ src, T *__restrict__ dst, uint32_t co, uint32_t ci,
    uint32_t slices, uint32_t nBlocks, uint64_t total, bool chansTransposed) {
  constexpr uint32_t E = 16 / sizeof(T);
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  const uint32_t e = uint32_t(tid % E), lane = uint32_t(tid / E) & 63;
  uint64_t r = tid / (64 * E);
  const uint32_t ks = uint32_t(r % slices);
  r /= slices;
  const uint32_t block = uint32_t(r % nBlocks);
  const uint64_t g = r / nBlocks;
  const uint32_t n = block * 32 + (lane & 31);
  const uint32_t k = ks * 2 * E + E * (lane >> 5) + e;
  // source [G][Co][Ci], or [G][Ci][Co] (a matrix multiplication's right-hand
  // side)
  dst[tid] = n >= co || k >= ci ? T(0)
             : chansTransposed  ? src[(g * ci + k) * co + n]
                                : src[(g * co + n) * ci + k];
}

/// Workgroups that share the pixel tiles of one (group, channel tile) pair:
/// as many workgroups as fit the chip at once (LDS allows 160 KB / ldsBytes
/// per CU), shared out over the pairs - and no more than give every walker
/// the same number of tiles (to within one): 3.1 tiles per walker would mean
/// a fourth round at a quarter of the chip.
uint64_t walkersFor(uint64_t mTiles, uint64_t pairs, uint32_t ldsBytes,
                    uint32_t cus) {
  const uint64_t resident = uint64_t(cus) * ((160 * 1024) / ldsBytes);
  uint64_t walkers = resident / pairs;
  if (walkers < 1)
    walkers = 1;
  const uint64_t tilesPerWalker = (mTiles + walkers - 1) / walkers;
  return (mTiles + tilesPerWalker - 1) / tilesPerWalker;
}

/// Tile height, ring depth and loader waves by input channels per group.
/// Tiles of 16 to 32 KB, a ring of three (one workgroup per CU), two or four
/// loader waves.  Measured on N = 32 layers of 56 x 56 (28 x 28 for 512
/// channels), against one loader wave and a ring of four (three for 512):
/// 64 -> 256 channels 15.9 against 19.3 us, 128 -> 128 10.1 against 11.2,
/// 256 -> 64 11.65 against 13.1, 512 -> 128 9.4 against 13.9.  One loader wave
/// does not issue a tile's loads - ten instructions each - as fast as HBM
/// delivers them; a deeper ring, or 128-pixel tiles where 64 are listed, is
/// slower.  512 channels: 64-pixel tiles (four compute waves, one on every
/// SIMD) in a ring of two, for layers that are as much the matrix cores' as
/// the memory's - against 32-pixel tiles in a ring of three, N = 32: 28 x 28,
/// 512 -> 512 21.8 -> 18.5 us, 512 -> 256 13.1 -> 11.3, 7 x 7, 512 -> 2048 8.3 ->
/// 7.3, 14 x 14, 512 -> 512 8.4 -> 7.6, but 28 x 28, 512 -> 128 8.8 -> 9.1.
struct PwShape {
  int tm, nb, lw;
};
constexpr PwShape kShape64{128, 3, 2}, kShape128{128, 3, 4},
    kShape256{64, 3, 2}, kShape512{64, 2, 4};
/// (`ci`: the layer's channels; rows of 16 and 32 channels take the shape of
/// 64: such layers are all output)
constexpr PwShape shapeFor(uint32_t ci) {
  return pwPaddedChans(ci) <= 64    ? kShape64
         : pwPaddedChans(ci) == 128 ? kShape128
         : pwPaddedChans(ci) == 256 ? kShape256
                                    : kShape512;
}
constexpr uint32_t ldsBytesOf(PwShape s, uint32_t ci, uint32_t nt = 1) {
  return uint32_t(s.nb * s.tm * (pwPaddedChans(ci) / 16) * 32 +
                  (s.tm / 16) * 32 * kPwStageRow + nt * kPwChans * 4);
}

/// 64-channel tiles of the output per workgroup.  With 64 input channels as
/// many (4, 3, 2, 1) as divide the layer's and still leave the chip two
/// workgroups per CU to share out.  With 128 input channels two, where every
/// workgroup still walks over six tiles or more: N = 32, 56 x 56, 128 -> 256
/// channels reads its 26 MB of input four times with one tile per workgroup
/// (25.1 us); on N = 32, 28 x 28, 128 -> 512 two tiles leave each workgroup
/// four pixel tiles instead of seven and lose (9.0 -> 10.6 us).
uint32_t chanTilesFor(const PointwiseDesc &d, uint32_t cus) {
  if (d.chanTiles)
    return d.chanTiles; // asked for by name (checked by pointwiseTakes)
  const PwShape s = shapeFor(pwRowChans(d));
  const uint64_t mTiles = (uint64_t(d.batch) * d.pixels + s.tm - 1) / s.tm;
  const uint64_t tiles64 = (d.outChansPerGroup + kPwChans - 1) / kPwChans;
  const uint32_t padded = pwPaddedChans(pwRowChans(d));
  if (padded <= 64) {
    for (uint32_t nt = 4; nt > 1; --nt)
      if (tiles64 % nt == 0 && mTiles * (tiles64 / nt) * d.groups >= 2ull * cus)
        return nt;
  } else if ((padded == 128 || padded == 256) && tiles64 % 2 == 0) {
    const uint64_t pairs = tiles64 / 2 * d.groups;
    const uint64_t walkers = walkersFor(
        mTiles, pairs, ldsBytesOf(s, pwRowChans(d), 2), cus);
    if ((mTiles + walkers - 1) / walkers >= 6)
      return 2;
  }
  return 1;
}

int deviceCUs() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) !=
            hipSuccess ||
        n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}

template <int KS, int TM, int NB, int LW, int NT, class OutT, int F>
hipError_t run(PwArgs a, const void *in, const void *w, const void *bias,
               void *out, hipStream_t stream) {
  constexpr int ldsBytes = ldsBytesOf(PwShape{TM, NB, LW}, KS * 16, NT);
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void *>(
          &pointwiseKernel<KS, TM, NB, LW, NT, OutT, F>),
      hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes);
  if (attr != hipSuccess)
    return attr;
  const int cus = deviceCUs();
  a.nTiles /= NT; // the workgroups' shares of NT * 64 channels
  a.mTiles = (a.M + TM - 1) / TM;
  const uint64_t pairs = uint64_t(a.nTiles) * a.d.groups;
  if (pairs == 0 || a.mTiles == 0)
    return hipSuccess;
  const uint64_t walkers = walkersFor(a.mTiles, pairs, ldsBytes, cus);
  a.walkers = uint32_t(walkers);
  const uint64_t blocks = walkers * pairs;
  // Tile indices up to mTiles + (NB - 1) * walkers are formed in 32 bits.
  if (blocks > 0x7fffffffull ||
      uint64_t(a.mTiles) + uint64_t(NB) * walkers > 0x7fffffffull / TM)
    return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((pointwiseKernel<KS, TM, NB, LW, NT, OutT, F>),
                     dim3(uint32_t(blocks)), dim3(TM * 4 + 64 * LW), ldsBytes,
                     stream, a, static_cast<const char *>(in),
                     static_cast<const char *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out));
  return hipGetLastError();
}

template <class OutT, int F>
hipError_t runSlices(const PwArgs &a, const void *in, const void *w,
                     const void *bias, void *out, hipStream_t stream) {
  const uint32_t nt = chanTilesFor(a.d, uint32_t(deviceCUs()));
  switch (pwPaddedChans(pwRowChans(a.d))) {
  case 16:
    if (nt == 4)
      return run<1, kShape64.tm, kShape64.nb, kShape64.lw, 4, OutT, F>(
          a, in, w, bias, out, stream);
    if (nt == 3)
      return run<1, kShape64.tm, kShape64.nb, kShape64.lw, 3, OutT, F>(
          a, in, w, bias, out, stream);
    if (nt == 2)
      return run<1, kShape64.tm, kShape64.nb, kShape64.lw, 2, OutT, F>(
          a, in, w, bias, out, stream);
    return run<1, kShape64.tm, kShape64.nb, kShape64.lw, 1, OutT, F>(
        a, in, w, bias, out, stream);
  case 32:
    if (nt == 4)
      return run<2, kShape64.tm, kShape64.nb, kShape64.lw, 4, OutT, F>(
          a, in, w, bias, out, stream);
    if (nt == 3)
      return run<2, kShape64.tm, kShape64.nb, kShape64.lw, 3, OutT, F>(
          a, in, w, bias, out, stream);
    if (nt == 2)
      return run<2, kShape64.tm, kShape64.nb, kShape64.lw, 2, OutT, F>(
          a, in, w, bias, out, stream);
    return run<2, kShape64.tm, kShape64.nb, kShape64.lw, 1, OutT, F>(
        a, in, w, bias, out, stream);
  case 64:
    if (nt == 4)
      return run<4, kShape64.tm, kShape64.nb, kShape64.lw, 4, OutT, F>(
          a, in, w, bias, out, stream);
    if (nt == 3)
      return run<4, kShape64.tm, kShape64.nb, kShape64.lw, 3, OutT, F>(
          a, in, w, bias, out, stream);
    if (nt == 2)
      return run<4, kShape64.tm, kShape64.nb, kShape64.lw, 2, OutT, F>(
          a, in, w, bias, out, stream);
    return run<4, kShape64.tm, kShape64.nb, kShape64.lw, 1, OutT, F>(
        a, in, w, bias, out, stream);
  case 128:
    if (nt == 2)
      return run<8, kShape128.tm, kShape128.nb, kShape128.lw, 2, OutT, F>(
          a, in, w, bias, out, stream);
    return run<8, kShape128.tm, kShape128.nb, kShape128.lw, 1, OutT, F>(
        a, in, w, bias, out, stream);
  case 256:
    if (nt == 2)
      return run<16, kShape256.tm, kShape256.nb, kShape256.lw, 2, OutT, F>(
          a, in, w, bias, out, stream);
    return run<16, kShape256.tm, kShape256.nb, kShape256.lw, 1, OutT, F>(
        a, in, w, bias, out, stream);
  case 512:
    return run<32, kShape512.tm, kShape512.nb, kShape512.lw, 1, OutT, F>(
        a, in, w, bias, out, stream);
  }
  return hipErrorInvalidValue;
}

} // namespace

bool pointwiseChanTilesOk(const PointwiseDesc &d, uint32_t chanTiles) {
  const uint32_t tiles64 = (d.outChansPerGroup + kPwChans - 1) / kPwChans;
  const uint32_t padded = pwPaddedChans(pwRowChans(d));
  const uint32_t most = padded <= 64 ? 4 : padded == 512 ? 1 : 2;
  return chanTiles >= 1 && chanTiles <= most && tiles64 % chanTiles == 0;
}

bool pointwiseTakes(const PointwiseDesc &d, int inType, int outType) {
  const uint32_t ci = d.inChansPerGroup, co = d.outChansPerGroup;
  const uint64_t m = uint64_t(d.batch) * d.pixels;
  const uint64_t inBytes = m * d.groups * ci * d.elemBytes;
  // fp16 (fp16 or fp32 out) or fp8 (fp16 out); rows of whole 16-byte
  // vectors, 1024 bytes at most
  const bool types =
      (inType == kHalf && d.elemBytes == 2 &&
       (outType == kHalf || outType == kFloat)) ||
      (inType == kQuarter && d.elemBytes == 1 && outType == kHalf);
  return types && ci != 0 && (ci * d.elemBytes) % 16 == 0 &&
         ci * d.elemBytes <= 1024 && co != 0 &&
         (d.chanTiles == 0 || pointwiseChanTilesOk(d, d.chanTiles)) &&
         co % (outType == kHalf ? 8 : 4) == 0 && m != 0 && m < 0x7fffffffull &&
         inBytes < kOutOfRange &&
         pointwisePackedElems(d) * d.elemBytes < kOutOfRange;
}

uint64_t pointwisePackedElems(const PointwiseDesc &d) {
  const uint64_t nBlocks = (d.outChansPerGroup + kPwChans - 1) / kPwChans * 2;
  // (1 KB per block and 32-byte k-slice)
  return uint64_t(d.groups) * nBlocks * (pwPaddedChans(pwRowChans(d)) / 16) *
         (1024 / d.elemBytes);
}

hipError_t launchPackPointwiseWeights(const PointwiseDesc &d, const void *src,
                                      void *dst, hipStream_t stream,
                                      bool chansTransposed) {
  const uint64_t total = pointwisePackedElems(d);
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const uint32_t nBlocks = (d.outChansPerGroup + kPwChans - 1) / kPwChans * 2;
  const uint32_t slices = pwPaddedChans(pwRowChans(d)) / 16;
  if (d.elemBytes == 2)
    hipLaunchKernelGGL(packPointwiseWeightsKernel<uint16_t>,
                       dim3(uint32_t(blocks)), dim3(256), 0, stream,
                       static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst), d.outChansPerGroup,
                       d.inChansPerGroup, slices, nBlocks, total,
                       chansTransposed);
  else
    hipLaunchKernelGGL(packPointwiseWeightsKernel<uint8_t>,
                       dim3(uint32_t(blocks)), dim3(256), 0, stream,
                       static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst), d.outChansPerGroup,
                       d.inChansPerGroup, slices, nBlocks, total,
                       chansTransposed);
  return hipGetLastError();
}

PointwiseLaunch pointwiseLaunchShape(const PointwiseDesc &d, uint32_t cus) {
  const PwShape s = shapeFor(pwRowChans(d));
  PointwiseLaunch l{};
  l.tilePixels = uint32_t(s.tm), l.ring = uint32_t(s.nb);
  l.loaderWaves = uint32_t(s.lw);
  const uint64_t mTiles = (uint64_t(d.batch) * d.pixels + s.tm - 1) / s.tm;
  const uint32_t nt = chanTilesFor(d, cus);
  l.chansPerWorkgroup = nt * kPwChans;
  const uint64_t pairs =
      uint64_t((d.outChansPerGroup + kPwChans - 1) / kPwChans) / nt * d.groups;
  if (mTiles == 0 || pairs == 0)
    return l;
  const uint64_t walkers =
      walkersFor(mTiles, pairs, ldsBytesOf(s, pwRowChans(d), nt), cus);
  l.workgroups = walkers * pairs;
  l.tilesPerWorkgroup = uint32_t((mTiles + walkers - 1) / walkers);
  return l;
}

hipError_t launchPointwise(const PointwiseDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, const QuarterInfo &q,
                           hipStream_t stream) {
  if (!pointwiseTakes(d, inType, outType))
    return hipErrorInvalidValue;
  PwArgs a;
  a.d = d;
  a.M = uint32_t(uint64_t(d.batch) * d.pixels);
  a.mTiles = 0; // set for the tile height of the kernel that runs
  a.nTiles = (d.outChansPerGroup + kPwChans - 1) / kPwChans;
  a.nBlocks = a.nTiles * 2;
  a.inBytes =
      uint32_t(uint64_t(a.M) * d.groups * d.inChansPerGroup * d.elemBytes);
  a.wBytes = uint32_t(pointwisePackedElems(d) * d.elemBytes);
  a.scale = inType == kQuarter ? q.scale : 1.0f;
  a.invScale = 1.0f / a.scale;
  if (inType == kQuarter) {
    const bool actsE5M2 = q.inFormat != kE4M3, wE5M2 = q.weightFormat != kE4M3;
    if (!actsE5M2 && !wE5M2)
      return runSlices<__half, 1>(a, in, weightsPacked, bias, out, stream);
    if (actsE5M2 && !wE5M2)
      return runSlices<__half, 2>(a, in, weightsPacked, bias, out, stream);
    if (!actsE5M2 && wE5M2)
      return runSlices<__half, 3>(a, in, weightsPacked, bias, out, stream);
    return runSlices<__half, 4>(a, in, weightsPacked, bias, out, stream);
  }
  if (outType == kHalf)
    return runSlices<__half, 0>(a, in, weightsPacked, bias, out, stream);
  return runSlices<float, 0>(a, in, weightsPacked, bias, out, stream);
}

} // namespace mxk

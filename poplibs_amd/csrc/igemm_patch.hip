// Implicit-GEMM forward convolution with the input patch of a tile resident
// in LDS: the kernel for unit-stride layers whose channels come in whole
// 128-byte slices (a ResNet-style 3x3 layer).
//
// Same GEMM view as igemm.hip (M = output pixels, N = output channels,
// K = taps x input channels), different data path.  A kernel of kH x kW taps
// reads every input element kH * kW times; igemm.hip fetches it through the
// vector cache that often, and at 64 bytes per clock that cache - not the
// matrix cores - bounds a 128 x 128 tile.  Here a workgroup loads the input
// rows its 128 output pixels read ONCE, zero padding materialised, and every
// tap's A operand is an LDS read at "pixel + tap offset": im2col is an
// address.  The weights never touch LDS: each wave owns 32 output channels and
// loads their MFMA operands straight into registers from a buffer packed in
// operand order, a few k-steps ahead.  So the loop has no barrier, no
// producer waves and no LDS writes, and the vector cache carries the weights
// only.
//
// Two kernels share this data path.  igemmPatchKernel (first in this file):
// MFMA 32x32, tiles of 32*RB pixels x 128 channels; wave (grp, wn) takes
// channels 32 wn .. 32 wn + 31 of all pixels, and of every k-step (128 bytes
// of K: one tap, one channel slice) the half `grp` - two waves per SIMD that
// cover each other's LDS latency, their sums meeting in LDS at the end.
// igemmPatch16Kernel (further down, with its own notes): MFMA 16x16, tiles of
// any height up to 112 pixels, the two waves of a SIMD taking k-steps in
// turn - what the planner picks.
//
// LDS patch: [slice][patch row][unit], a unit = 16 bytes, a pixel = 8 units
// of channels + 1 or 2 unused: at a pitch of 144 bytes (32-pixel MFMA blocks)
// or 160 bytes (16-pixel blocks) the 16-byte operand reads of neighbouring
// pixels cover all 64 banks without any swizzle, so a tap is a plain byte
// offset.  A patch row = the input row of one image with its zero padding
// left and right; the pitch of the rows continues the pixels' progression
// through the banks (modulo 256 bytes).  Patch rows are the rows, padding
// rows included, of consecutive images that the tile's pixels read.
//
// Takes the role of PopLibs' AMP vertex ConvPartialnx1
// (lib/poplin/codelets/ConvPartialnx1.cpp:52-246) for these shapes; the fp8
// scale 2^(sIn + sW) is applied once to the fp32 sum
// (lib/poplin/codelets/inlineAssemblerConv.hpp:28-33).
#include "igemm_common.hpp"

#include <algorithm>

namespace mxk {
namespace {

#ifndef PATCH_TN
#define PATCH_TN 1
#endif
// 32-channel blocks per wave; the tile's 128 channels take kWavesN waves, and
// as many again for the other half of K.
constexpr int kTN = PATCH_TN;
constexpr int kWavesN = 4 / kTN;
constexpr int kPatchWaves = 2 * kWavesN;
constexpr int kPatchThreads = 64 * kPatchWaves;
// 16-byte units per pixel in the patch: 8 of channels and padding that keeps
// the MFMA operand reads free of bank conflicts - 144 bytes from pixel to
// pixel where 32 lanes read 32 pixels (igemmPatchKernel), 160 bytes where 16
// lanes read 16 (igemmPatch16Kernel; measured: 246 bytes per clock against
// 171 at 144).
constexpr int kPixelUnits = 9, kPixelUnits16 = 10;
constexpr int kPatchBN = 128;
constexpr int kLdsLimit = 160 * 1024;
// An offset no buffer the kernel makes reaches: marks padding rows / columns.
constexpr uint32_t kInvalid = 0x40000000u;

// Cycle stamps of igemmPatch16Kernel's phases, for the build with
// -DMXK_PATCH_STAMPS only (libmxconv_stamps.so; the product library carries
// none of this).  Waves 0 and 4 of every workgroup - the older and the younger
// wave of SIMD 0 - write s_memtime at the marked points, and the wall clock
// (s_memrealtime, 100 MHz) at both ends, to the buffer
// mxk_patch_stamp_sink() names: [workgroup][wave 0 | 4][kStampSlots] of 8
// bytes.
#ifdef MXK_PATCH_STAMPS
constexpr int kStampSlots = 16;
__device__ uint64_t *patchStampSink = nullptr;
#define MXK_STAMP_DECL uint64_t stamps_[kStampSlots] = {}
#define MXK_STAMP(i) stamps_[i] = __builtin_amdgcn_s_memtime()
#define MXK_STAMP_REAL(i) stamps_[i] = __builtin_amdgcn_s_memrealtime()
#define MXK_STAMP_ARG , stamps_
#define MXK_STAMP_PARAM , uint64_t *stamps_
#else
#define MXK_STAMP_DECL
#define MXK_STAMP(i)
#define MXK_STAMP_REAL(i)
#define MXK_STAMP_ARG
#define MXK_STAMP_PARAM
#endif

struct PatchArgs {
  uint32_t M, mTiles, nTiles, groups;
  uint32_t tileM; // output pixels per tile
  uint32_t outW, outH;
  uint32_t rowsPerImage; // patch rows per image: outH + (kH - 1) * dilH
  uint32_t inH;
  int32_t padH, padW;
  uint32_t loH, spanH, loW, spanW;
  uint32_t kW, taps, slices, kSteps;
  uint32_t tapRowBytes, tapColBytes; // LDS bytes per kernel row / column
  uint32_t rowLoads;   // wave loads (1 KB, the last one partial) per patch row
  uint32_t rowUnits;   // units of a patch row
  uint32_t rowPitch;   // LDS bytes from one patch row to the next
  uint32_t sliceBytes; // LDS bytes of one channel slice of the patch
  uint32_t exchangeByte, tileByte; // where the epilogue keeps its data in LDS
  uint32_t pixelBytes, ciBytes, inRowBytes, imageBytes;
  uint64_t inBytes;
  uint32_t outChans, outChansPerGroup;
  uint32_t wBytes;
  FastDiv divOutW, divOutH, divNTiles, divMTiles, divRowLoads, divRowsPerImage;
  FastDiv divTaps, divKW;
};

/// LDS the reduction of the two K halves and the output tile need.
template <int RB, class OutT> constexpr int patchEpilogueBytes() {
  return kPatchWaves * (RB / 2) * kTN * 4 * 1024 +
         32 * RB * (kPatchBN * int(sizeof(OutT)) + 16);
}

/// The output pixels [m0, mLast] of a tile and the patch rows they read: rows
/// [firstRow, firstRow + rows) of the sequence "image 0's rowsPerImage padded
/// rows, image 1's, ...".
struct TileSpan {
  uint32_t m0, mLast, image0, firstRow, rows;
};

__device__ __forceinline__ TileSpan tileSpan(const PatchArgs &a,
                                             uint32_t mTile) {
  TileSpan s;
  s.m0 = mTile * a.tileM;
  s.mLast = (s.m0 + a.tileM < a.M ? s.m0 + a.tileM : a.M) - 1;
  const uint32_t q0 = a.divOutW(s.m0);
  s.image0 = a.divOutH(q0);
  s.firstRow = s.image0 * a.rowsPerImage + (q0 - s.image0 * a.outH);
  const uint32_t qL = a.divOutW(s.mLast), imageL = a.divOutH(qL);
  s.rows = imageL * a.rowsPerImage + (qL - imageL * a.outH) +
           (a.rowsPerImage - a.outH) + 1 - s.firstRow;
  return s;
}

/// LDS byte of output pixel m's tap (0, 0) in slice 0 of the patch.
template <int UNITS>
__device__ __forceinline__ uint32_t patchByteOf(const PatchArgs &a,
                                                const TileSpan &s, uint32_t m) {
  m = m < s.mLast ? m : s.mLast;
  const uint32_t q = a.divOutW(m), ow = m - q * a.outW;
  const uint32_t image = a.divOutH(q), oh = q - image * a.outH;
  return (image * a.rowsPerImage + oh - s.firstRow) * a.rowPitch +
         ow * (16 * UNITS);
}

/// Loads the patch of a tile, all waves together.  Column blocks of all
/// slices, slice 0 first, are dealt out to the waves in turn.  Slice 0 is what
/// the k loop waits for: its loads go out before anything else, then
/// `between()` runs (the first weight loads - WEIGHT_LOADS of them per wave -
/// and address arithmetic, which fill the wait), then the wave waits for its
/// part of slice 0 and meets the others at a barrier; the later slices' loads
/// follow and are waited for inside the k loop.
template <int WEIGHT_LOADS, int UNITS, class Between, class Behind>
__device__ __forceinline__ void
loadPatch(const PatchArgs &a, const char *__restrict__ in, char *lds, int wave,
          int lane, uint32_t g, const TileSpan &span, Between &&between,
          Behind &&behind MXK_STAMP_PARAM) {
  // Patch row `lane`: where its input row starts, from the first image the
  // tile reads (32-bit offsets), or kInvalid for a row of padding.  A load
  // adds the lane's own offset, itself kInvalid for padding columns: any sum
  // with a kInvalid in it lies beyond the buffer, which the range check
  // limits to kInvalid bytes, and reads as zeros.
  uint32_t rowBase;
  {
    const uint32_t r = span.firstRow + lane;
    const uint32_t image = a.divRowsPerImage(r);
    const uint32_t ih = r - image * a.rowsPerImage - uint32_t(a.padH);
    rowBase = ih - a.loH < a.spanH
                  ? ((image - span.image0) * a.inH + ih) * a.inRowBytes +
                        g * a.ciBytes
                  : kInvalid;
  }
  const uint64_t skipped = uint64_t(span.image0) * a.imageBytes;
  const uint64_t left = a.inBytes - skipped;
  const __amdgpu_buffer_rsrc_t inBuf =
      bufferOf(in + skipped, uint32_t(left < kInvalid ? left : kInvalid));
  const uint32_t rows = span.rows;
  // One wave loads column block q (units 64 q .. 64 q + 63 of every patch
  // row: chunk u % UNITS of the pixel in padded column u / UNITS) of a
  // slice.
  auto loadColumns = [&](uint32_t slice, uint32_t q) {
    const uint32_t u = q * 64 + lane;
    const uint32_t col = u / UNITS, c = u - col * UNITS;
    const uint32_t iw = col - uint32_t(a.padW);
    const uint32_t laneOff =
        c < 8 && iw - a.loW < a.spanW ? iw * a.pixelBytes + c * 16 : kInvalid;
    // (the last block of a row is a partial one: lanes beyond it write
    // nothing)
    if (u < a.rowUnits) {
      char *dst = lds + slice * a.sliceBytes + q * 1024;
      auto loadRow = [&](uint32_t row) {
        const uint32_t base = __builtin_amdgcn_readlane(rowBase, row);
        loadToLds(inBuf, (LdsPtr)dst, laneOff + base, slice * 128);
        dst += a.rowPitch;
      };
      // (four at a time: a taken branch costs as much as a load)
      uint32_t row = 0;
      for (; row + 4 <= rows; row += 4) {
        loadRow(row), loadRow(row + 1), loadRow(row + 2), loadRow(row + 3);
      }
      for (; row < rows; ++row)
        loadRow(row);
    }
  };
  // A wave with no block of slice 0 issues its first block of a later slice
  // right away (behind `between`, so that slice 0 gets ahead); the others do
  // so after the barrier.
  MXK_STAMP(1); // set-up done: the first load of the patch goes out
  const uint32_t blocks = a.slices * a.rowLoads;
  uint32_t next = wave;
  for (; next < a.rowLoads; next += kPatchWaves)
    loadColumns(0, next);
  MXK_STAMP(2); // slice 0 requested
  const bool early = uint32_t(wave) >= a.rowLoads;
  between();
  MXK_STAMP(3); // first weights requested, pixel offsets worked out
  if (early) {
    if (next < blocks) {
      const uint32_t s = a.divRowLoads(next);
      loadColumns(s, next - s * a.rowLoads);
      next += kPatchWaves;
    }
  } else {
    // slice 0 is in LDS once all but the weight loads have landed
    MXK_WAIT_VMCNT(WEIGHT_LOADS);
  }
  MXK_STAMP(4); // own part of slice 0 landed
  __builtin_amdgcn_s_barrier();
  MXK_STAMP(5); // everybody's has
  behind();
  // What is left of the later slices goes to the older wave of each SIMD
  // (waves 0 .. kWavesN - 1): it wins the MFMA slots, is through its k-steps
  // long before the younger one and waits for it at the end, while the
  // kernel's end waits for the younger one - which so enters the k loop
  // without standing in the queue of the vector memory path (22 cycles per
  // load of 1 KB: 1 600 cycles for three slices of a 112-pixel tile).
  // Issued so far: slice 0's blocks and one block per wave without any.
  if (wave < kWavesN) {
    const uint32_t issued =
        a.rowLoads > uint32_t(kPatchWaves) ? a.rowLoads : uint32_t(kPatchWaves);
    for (next = issued + wave; next < blocks; next += kWavesN) {
      const uint32_t s = a.divRowLoads(next);
      loadColumns(s, next - s * a.rowLoads);
    }
  }
}

/// The finished tile, [row][128 channels] at a pitch of kOutRow bytes in LDS,
/// goes out as 16-byte stores, whole rows per instruction, through a buffer
/// that ends with the last valid row: rows beyond it go nowhere.  (Written
/// through the L2: nothing is left to write back when the kernel ends.)
/// ROWS: rows the tile has room for in LDS.
template <int ROWS, class OutT>
__device__ __forceinline__ void
storeTile(const PatchArgs &a, const char *tileOut, OutT *__restrict__ out,
          int t, uint32_t g, uint32_t nTile, const TileSpan &span) {
  constexpr int kOutRow = kPatchBN * int(sizeof(OutT)) + 16;
  constexpr int kVecsPerRow = kPatchBN * int(sizeof(OutT)) / 16;
  constexpr int kRowsPerPass = kPatchThreads / kVecsPerRow;
  static_assert(ROWS % kRowsPerPass == 0, "whole passes");
  const uint32_t outRowBytes = a.outChans * sizeof(OutT);
  const uint32_t validRows = span.mLast + 1 - span.m0;
  const uint32_t nLeft = a.outChansPerGroup - nTile * kPatchBN;
  const uint32_t validBytes =
      (nLeft < uint32_t(kPatchBN) ? nLeft : kPatchBN) * sizeof(OutT);
  const __amdgpu_buffer_rsrc_t outBuf = bufferOf(
      out + size_t(span.m0) * a.outChans + g * a.outChansPerGroup +
          nTile * kPatchBN,
      (validRows - 1) * outRowBytes + validBytes);
  const uint32_t row = t / kVecsPerRow, vecByte = (t % kVecsPerRow) * 16;
  const uint32_t to =
      vecByte < validBytes ? row * outRowBytes + vecByte : kOutOfRange;
  const char *from = tileOut + row * kOutRow + vecByte;
#pragma unroll
  for (int pass = 0; pass != ROWS / kRowsPerPass; ++pass)
    __builtin_amdgcn_raw_buffer_store_b128(
        *reinterpret_cast<const uintx4 *>(from +
                                          pass * kRowsPerPass * kOutRow),
        outBuf, to, pass * kRowsPerPass * outRowBytes, kWriteThroughStore);
}

template <int EB> struct PatchMma;
/// fp16: a wave's half of a k-step is two MFMAs of K = 16 per row block; lane
/// l holds row l % 32, 8 consecutive k from 8 (l / 32) of the MFMA's 16.
template <> struct PatchMma<2> {
  // byte offset inside the 128-byte slice of what lane half h reads for
  // sub-step j of K half grp
  static __device__ __forceinline__ int laneByte(int grp, int h) {
    return grp * 64 + h * 16;
  }
  static constexpr int kSubBytes = 32; // from sub-step 0 to sub-step 1
  static constexpr int kPasses = 2;     // MFMAs per row block and k-step half
  template <int P, int FA, int FB>
  static __device__ __forceinline__ void
  mul(const uintx4 (&b)[2], const uintx4 (&a0), const uintx4 (&a1),
      floatx16 &acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(
        __builtin_bit_cast(half8, b[P]),
        __builtin_bit_cast(half8, P == 0 ? a0 : a1), acc, 0, 0, 0);
  }
};
/// fp8: a wave's half of a k-step is one MFMA of K = 64 per row block; lane l
/// holds row l % 32, 32 consecutive bytes from 32 (l / 32).
template <> struct PatchMma<1> {
  static __device__ __forceinline__ int laneByte(int grp, int h) {
    return grp * 64 + h * 32;
  }
  static constexpr int kSubBytes = 16;
  static constexpr int kPasses = 1;
  template <int P, int FA, int FB>
  static __device__ __forceinline__ void
  mul(const uintx4 (&b)[2], const uintx4 (&a0), const uintx4 (&a1),
      floatx16 &acc) {
    const intx8 bb{int(b[0].x), int(b[0].y), int(b[0].z), int(b[0].w),
                   int(b[1].x), int(b[1].y), int(b[1].z), int(b[1].w)};
    const intx8 aa{int(a0.x), int(a0.y), int(a0.z), int(a0.w),
                   int(a1.x), int(a1.y), int(a1.z), int(a1.w)};
    acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bb, aa, acc, FB, FA,
                                                          0, 0, 0, 0);
  }
};

/// EB: bytes per input element (2 half, 1 quarter); FA / FB: fp8 formats of
/// activations / weights; RB: 32-row blocks per tile; D: k-steps the weight
/// loads run ahead.
template <int EB, int FA, int FB, int RB, int D, class OutT>
__global__ __launch_bounds__(kPatchThreads) void igemmPatchKernel(
    const PatchArgs a, const char *__restrict__ in, const char *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out, float scale) {
  constexpr int BM = 32 * RB;
  constexpr int H = RB / 2; // row blocks a wave finishes
  extern __shared__ __align__(16) char lds[];
  using Mma = PatchMma<EB>;
  MXK_STAMP_DECL; // (only igemmPatch16Kernel writes them out)

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int grp = wave / kWavesN, wn = wave % kWavesN;

  const uint32_t tile = xcdSwizzle(blockIdx.x, gridDim.x);
  const uint32_t overN = a.divNTiles(tile);
  const uint32_t nTile = tile - overN * a.nTiles;
  const uint32_t g = a.divMTiles(overN);
  const uint32_t mTile = overN - g * a.mTiles;
  const TileSpan span = tileSpan(a, mTile);

  // The weights of this wave's 32 kTN channels: per k-step and K half 2 KB per
  // 32 channels, lane l's two 16-byte operands at 16 l and 1024 + 16 l; the
  // two halves of a step follow each other.  The buffer ends with the wave's
  // share of the last step, so the loads that run ahead beyond it read zeros.
  constexpr uint32_t kShare = kTN * 2048, kStepBytes = 2 * kShare;
  const uint32_t waveBlock = (g * a.nTiles + nTile) * kWavesN + wn;
  const __amdgpu_buffer_rsrc_t wBuf =
      bufferOf(w + (size_t(waveBlock) * a.kSteps * 2 + grp) * kShare,
               (a.kSteps - 1) * kStepBytes + kShare);
  uint32_t wOff = lane * 16;
  uintx4 bf[D][kTN][2];
  auto loadB = [&](uintx4(&dst)[kTN][2]) {
#pragma unroll
    for (int c = 0; c != kTN; ++c)
#pragma unroll
      for (int j = 0; j != 2; ++j)
        dst[c][j] = __builtin_bit_cast(
            uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                        wBuf, wOff + c * 2048 + j * 1024, 0, 0));
    wOff += kStepBytes;
  };

  // Per row block: the LDS byte of the first chunk this lane reads of a
  // k-step, at tap (0, 0) of slice 0.  (Worked out while the first loads are
  // in flight.)
  uint32_t pixelByte[RB];
  loadPatch<2 * kTN * D, kPixelUnits>(a, in, lds, wave, lane, g, span, [&] {
#pragma unroll
    for (int u = 0; u != D; ++u)
      loadB(bf[u]);
#pragma unroll
    for (int i = 0; i != RB; ++i)
      pixelByte[i] =
          patchByteOf<kPixelUnits>(a, span, span.m0 + i * 32 + (lane & 31)) +
                     Mma::laneByte(grp, lane >> 5);
    // (keeps the arithmetic above this point: it fills the wait)
#pragma unroll
    for (int i = 0; i != RB; ++i)
      asm volatile("" ::"v"(pixelByte[i]));
  }, [] {} MXK_STAMP_ARG);

  floatx16 acc[RB][kTN];
#pragma unroll
  for (int i = 0; i != RB; ++i)
#pragma unroll
    for (int c = 0; c != kTN; ++c)
#pragma unroll
      for (int v = 0; v != 16; ++v)
        acc[i][c][v] = 0.0f;

  // k-step kt = slice * taps + tap; its A operands sit at pixelByte + tapByte.
  // The offsets of 64 steps at a time are kept one per lane: lane j holds
  // step tableBase + 1 + j's, with bit 31 set on the first tap of a slice.
  uint32_t tapByte = 0, tapTable = 0, tableBase = 0;
  auto fillTable = [&] {
    const uint32_t kt = tableBase + 1 + lane;
    const uint32_t slice = a.divTaps(kt), tap = kt - slice * a.taps;
    const uint32_t kh = a.divKW(tap), kw = tap - kh * a.kW;
    tapTable = (slice * a.sliceBytes + kh * a.tapRowBytes +
                kw * a.tapColBytes) |
               (tap == 0 ? 0x80000000u : 0u);
  };
  fillTable();
  struct Operands {
    uintx4 lo[RB], hi[RB];
  };
  auto readA = [&](Operands &x) {
    // (in the order the MFMAs take them)
#pragma unroll
    for (int i = 0; i != RB; ++i)
      x.lo[i] =
          *reinterpret_cast<const uintx4 *>(lds + pixelByte[i] + tapByte);
#pragma unroll
    for (int i = 0; i != RB; ++i)
      x.hi[i] = *reinterpret_cast<const uintx4 *>(lds + pixelByte[i] +
                                                  tapByte + Mma::kSubBytes);
  };
  // (MFMAs into one accumulator depend on each other: the other row blocks'
  // go in between)
  auto multiply = [&](const uintx4(&b)[kTN][2], const Operands &x) {
    staticFor<0, Mma::kPasses>([&](auto pass) {
#pragma unroll
      for (int i = 0; i != RB; ++i)
#pragma unroll
        for (int c = 0; c != kTN; ++c)
          Mma::template mul<decltype(pass)::value, FA, FB>(
              b[c], x.lo[i], x.hi[i], acc[i][c]);
    });
  };
  // One k-step.  The LDS reads of the next step and the weight load that
  // reuses this step's registers are dealt out between this step's MFMAs: a
  // wave issues in order, and an MFMA behind another waits for the pipe, so
  // whatever stands between two of them costs nothing.
  // GUARD: the steps behind the last whole group of D.
  auto step = [&](auto guard, uintx4(&b)[kTN][2], const Operands &cur,
                  Operands &next, uint32_t kt) {
    constexpr bool GUARD = decltype(guard)::value;
    const bool more = !GUARD || kt + 1 < a.kSteps;
    if (more) {
      const uint32_t entry =
          __builtin_amdgcn_readlane(tapTable, kt - tableBase);
      tapByte = entry & 0x7fffffffu;
      if (entry & 0x80000000u) {
        // A new slice: its loads were issued before the loop, so they are
        // older than the weight loads of the last D steps (loads complete in
        // order); the barrier tells that the other waves' have landed too.
        if (kt >= uint32_t(D))
          MXK_WAIT_VMCNT(2 * kTN * (D - 1));
        else
          MXK_WAIT_VMCNT(0);
        __builtin_amdgcn_s_barrier();
      }
    }
    if constexpr (!GUARD) {
      readA(next);
      multiply(b, cur);
      loadB(b);
      // address arithmetic first, then MFMA and LDS read in turn, the weight
      // loads behind the last MFMAs
      __builtin_amdgcn_sched_group_barrier(0x002, RB, 0);
      constexpr int kMfmas = Mma::kPasses * RB * kTN;
      constexpr int kPerRead = kMfmas / (2 * RB) ? kMfmas / (2 * RB) : 1;
      constexpr int kReads = kMfmas / kPerRead;
#pragma unroll
      for (int k = 0; k != kReads; ++k) {
        __builtin_amdgcn_sched_group_barrier(0x008, kPerRead, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * RB / kReads, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x020, 2 * kTN, 0);
    } else {
      if (more)
        readA(next);
      if (kt < a.kSteps)
        multiply(b, cur);
    }
  };
  static_assert(D % 2 == 0, "the operand buffers alternate");
  Operands even, odd;
  // (nothing but these LDS reads pending at the head of the loop, so that
  // the waits inside it count reads)
  MXK_WAIT_LGKMCNT0();
  readA(even);
  uint32_t kt = 0;
  // (every step of a whole group has a successor to fetch for: the last
  // steps, at least one, are left to the guarded group)
  for (; kt + D < a.kSteps; kt += D) {
    if (kt - tableBase == 64) {
      tableBase = kt;
      fillTable();
    }
#pragma unroll
    for (int u = 0; u != D; u += 2) {
      step(std::false_type{}, bf[u], even, odd, kt + u);
      step(std::false_type{}, bf[u + 1], odd, even, kt + u + 1);
    }
  }
  {
    if (kt - tableBase == 64) {
      tableBase = kt;
      fillTable();
    }
#pragma unroll
    for (int u = 0; u != D; u += 2) {
      step(std::true_type{}, bf[u], even, odd, kt + u);
      step(std::true_type{}, bf[u + 1], odd, even, kt + u + 1);
    }
  }

  // Sum the two K halves: a wave keeps H of its row blocks and hands the
  // others to the wave with the same channels and the other K half, through
  // LDS - beside the patch where there is room, else in its place, once
  // everybody is done with it.
  if (a.exchangeByte == 0)
    __syncthreads();
  {
    uintx4 *exchange = reinterpret_cast<uintx4 *>(lds + a.exchangeByte);
    constexpr int kOutRow = kPatchBN * int(sizeof(OutT)) + 16;
    constexpr int kGive = H * kTN * 4; // 16-byte vectors a lane hands over
    char *tileOut = lds + a.tileByte;
    // (the K half as a compile-time number: the accumulators are registers
    // and want constant indices)
    auto give = [&](auto half) {
      constexpr int G = decltype(half)::value;
#pragma unroll
      for (int i = 0; i != H; ++i)
#pragma unroll
        for (int c = 0; c != kTN; ++c)
#pragma unroll
          for (int v = 0; v != 4; ++v) {
            const floatx16 &x = acc[(1 - G) * H + i][c];
            exchange[((wn * 2 + (1 - G)) * kGive + (i * kTN + c) * 4 + v) *
                         64 +
                     lane] =
                __builtin_bit_cast(uintx4, floatx4{x[4 * v], x[4 * v + 1],
                                                   x[4 * v + 2], x[4 * v + 3]});
          }
    };
    if (grp == 0)
      give(std::integral_constant<int, 0>{});
    else
      give(std::integral_constant<int, 1>{});
    __syncthreads();
    const uint32_t nLane = wn * 32 * kTN + (lane >> 5) * 4;
    // the lane's channels of the tile are nLane + 32 c + 8 q + e, q, e < 4
    char *laneOut = tileOut + (lane & 31) * kOutRow + nLane * sizeof(OutT);
    const char *laneIn =
        lds + a.exchangeByte +
        ((wn * 2 + grp) * kGive * 64 + lane) * sizeof(uintx4);
    auto keep = [&](auto half, auto biased) {
      constexpr int G = decltype(half)::value;
      float bv[kTN][4][4];
      if constexpr (decltype(biased)::value) {
        // (the channel count is a multiple of the output vector, so a run of
        // four channels is inside it or outside)
#pragma unroll
        for (int c = 0; c != kTN; ++c)
#pragma unroll
        for (int q = 0; q != 4; ++q) {
          const uint32_t n = nTile * kPatchBN + nLane + 32 * c + 8 * q;
          const OutT *b = bias + g * a.outChansPerGroup +
                          (n < a.outChansPerGroup ? n : 0);
          if constexpr (sizeof(OutT) == 2) {
            const uint2 raw = *reinterpret_cast<const uint2 *>(b);
            const __half2 lo = __builtin_bit_cast(__half2, raw.x),
                          hi = __builtin_bit_cast(__half2, raw.y);
            bv[c][q][0] = __low2float(lo), bv[c][q][1] = __high2float(lo);
            bv[c][q][2] = __low2float(hi), bv[c][q][3] = __high2float(hi);
          } else {
            const float4 raw = *reinterpret_cast<const float4 *>(b);
            bv[c][q][0] = raw.x, bv[c][q][1] = raw.y, bv[c][q][2] = raw.z,
            bv[c][q][3] = raw.w;
          }
        }
      }
      floatx4 other[H][kTN][4];
#pragma unroll
      for (int i = 0; i != H; ++i)
#pragma unroll
        for (int c = 0; c != kTN; ++c)
#pragma unroll
          for (int q = 0; q != 4; ++q)
            other[i][c][q] = *reinterpret_cast<const floatx4 *>(
                laneIn + ((i * kTN + c) * 4 + q) * 1024);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i != H; ++i)
#pragma unroll
        for (int c = 0; c != kTN; ++c)
#pragma unroll
          for (int q = 0; q != 4; ++q) {
            float v[4];
#pragma unroll
            for (int e = 0; e != 4; ++e) {
              v[e] = acc[G * H + i][c][4 * q + e] + other[i][c][q][e];
              if constexpr (EB == 1)
                v[e] *= scale;
              if constexpr (decltype(biased)::value)
                v[e] += bv[c][q][e];
            }
            storeOut4(reinterpret_cast<OutT *>(laneOut +
                                               (G * H + i) * 32 * kOutRow) +
                          32 * c + 8 * q,
                      v);
          }
    };
    if (bias) {
      if (grp == 0)
        keep(std::integral_constant<int, 0>{}, std::true_type{});
      else
        keep(std::integral_constant<int, 1>{}, std::true_type{});
    } else {
      if (grp == 0)
        keep(std::integral_constant<int, 0>{}, std::false_type{});
      else
        keep(std::integral_constant<int, 1>{}, std::false_type{});
    }
    __syncthreads();
    storeTile<BM>(a, tileOut, out, t, g, nTile, span);
  }
}

// ---------------------------------------------------------------------------
// The same kernel on 16-pixel MFMA blocks, for tiles of any height up to 112
// pixels: a layer of M pixels is cut into as many equal tiles as there are
// CUs (the 25 088 pixels of a 32 x 28 x 28 layer: 256 tiles of 98 instead of
// 196 of 128), and seven 16-row blocks cover the tile with less padding than
// four 32-row ones would.  Differences from the kernel above:
//   - MFMA 16x16x32 (fp16) / 16x16x128 (fp8): a wave's 32 channels are two
//     column blocks, so an A operand read from LDS feeds two MFMAs;
//   - the two waves of a SIMD split K by k-step parity (wave grp takes steps
//     grp, grp + 2, ...) - an fp8 MFMA spans a whole 128-byte k-step;
//   - packed weights: [group][32 channels][k-step][4 operands][lane][16 B],
//     operand (u, c) = K unit u (64 bytes of K), column block c for fp16;
//     (c, r) = column block c, 16-byte half r of the lane's 32 bytes for fp8;
//     lane l holds channel 16 c + l % 16 and the K bytes the A side's lane l
//     reads (16 (l / 16) of the unit; 64 r + 16 (l / 16) of the step).
// ---------------------------------------------------------------------------
constexpr int kAhead16 = 2; // own k-steps the weight loads run ahead
constexpr int kBlocks16 = 7;              // 16-row blocks per tile
constexpr int kRows16 = 16 * kBlocks16;   // pixels a tile has room for
constexpr int kKeep16 = (kBlocks16 + 1) / 2; // blocks K half 0's wave finishes

template <int EB> struct PatchMma16;
template <> struct PatchMma16<2> {
  static constexpr int kUnits = 2; // MFMA K = 32 halves: two per k-step
  static constexpr int kReads = 1; // 16-byte operands per lane and MFMA
  static __device__ __forceinline__ int laneByte(int quarter) {
    return quarter * 16;
  }
  template <int FA, int FB>
  static __device__ __forceinline__ void
  mul(const uintx4 (&b)[kReads], const uintx4 (&x)[kReads], floatx4 &acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(
        __builtin_bit_cast(half8, b[0]), __builtin_bit_cast(half8, x[0]), acc,
        0, 0, 0);
  }
};
template <> struct PatchMma16<1> {
  static constexpr int kUnits = 1; // MFMA K = 128 bytes: the k-step
  // Two 16-byte reads per lane, 64 bytes apart: each of them then has the
  // fp16 read's pattern (which K bytes a lane multiplies does not matter as
  // long as the weights are packed alike).
  static constexpr int kReads = 2;
  static __device__ __forceinline__ int laneByte(int quarter) {
    return quarter * 16;
  }
  template <int FA, int FB>
  static __device__ __forceinline__ void
  mul(const uintx4 (&b)[kReads], const uintx4 (&x)[kReads], floatx4 &acc) {
    const intx8 bb{int(b[0].x), int(b[0].y), int(b[0].z), int(b[0].w),
                   int(b[1].x), int(b[1].y), int(b[1].z), int(b[1].w)};
    const intx8 xx{int(x[0].x), int(x[0].y), int(x[0].z), int(x[0].w),
                   int(x[1].x), int(x[1].y), int(x[1].z), int(x[1].w)};
    acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bb, xx, acc, FB, FA,
                                                           0, 0, 0, 0);
  }
};

/// D: k-steps of its own (every second one) a wave's weight loads run ahead.
template <int EB, int FA, int FB, int D, class OutT>
__global__ __launch_bounds__(kPatchThreads) void igemmPatch16Kernel(
    const PatchArgs a, const char *__restrict__ in, const char *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out, float scale) {
  static_assert(kTN == 1 && D % 2 == 0 && 64 % D == 0, "");
  constexpr int RB = kBlocks16;
  extern __shared__ __align__(16) char lds[];
  using Mma = PatchMma16<EB>;
  constexpr int kUnits = Mma::kUnits, kReads = Mma::kReads;
  MXK_STAMP_DECL;
  MXK_STAMP_REAL(14);
  MXK_STAMP(0);

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int grp = wave / kWavesN, wn = wave % kWavesN;

  const uint32_t tile = xcdSwizzle(blockIdx.x, gridDim.x);
  // (Arguments the compiler would otherwise fetch where they are first used,
  // each fetch a round trip of the scalar cache on the way to the first MFMA:
  // naming them here puts them into the one fetch at the kernel's start.)
  asm volatile("" ::"s"(w), "s"(out), "s"(bias), "s"(a.inH), "s"(a.ciBytes),
               "s"(a.inRowBytes), "s"(a.outChans), "s"(a.outChansPerGroup));
  const uint32_t overN = a.divNTiles(tile);
  const uint32_t nTile = tile - overN * a.nTiles;
  const uint32_t g = a.divMTiles(overN);
  const uint32_t mTile = overN - g * a.mTiles;
  const TileSpan span = tileSpan(a, mTile);

  // This wave's k-steps: grp, grp + 2, ... - `own` of them (at least one: the
  // kernel has two taps or more).  Their weights: 4 KB per step, lane l's four
  // operands 1 KB apart; the buffer ends with the wave's last step, so the
  // loads that run ahead beyond it read zeros.
  const uint32_t own = (a.kSteps + 1 - grp) >> 1;
  const uint32_t waveBlock = (g * a.nTiles + nTile) * kWavesN + wn;
  const __amdgpu_buffer_rsrc_t wBuf =
      bufferOf(w + (size_t(waveBlock) * a.kSteps + grp) * 4096,
               (own - 1) * 8192 + 4096);
  uint32_t wOff = lane * 16;
  uintx4 bf[D][kUnits][2][kReads];
  auto loadB = [&](uintx4(&dst)[kUnits][2][kReads]) {
#pragma unroll
    for (int u = 0; u != kUnits; ++u)
#pragma unroll
      for (int c = 0; c != 2; ++c)
#pragma unroll
        for (int r = 0; r != kReads; ++r)
          dst[u][c][r] = __builtin_bit_cast(
              uintx4,
              __builtin_amdgcn_raw_buffer_load_b128(
                  wBuf, wOff + ((u * 2 + c) * kReads + r) * 1024, 0, 0));
    wOff += 8192;
  };

  // Per row block: the LDS byte of the first chunk this lane reads of a
  // k-step, at tap (0, 0) of slice 0.
  uint32_t pixelByte[RB];
  // (the first step's weights before the barrier, the others behind it: the
  // vector memory path is what bounds the time to the barrier)
  constexpr int kFirst = 1;
  loadPatch<4 * kFirst, kPixelUnits16>(a, in, lds, wave, lane, g, span, [&] {
#pragma unroll
    for (int u = 0; u != kFirst; ++u)
      loadB(bf[u]);
    // Lane l works out where pixels l and 64 + l of the tile sit in the
    // patch (two divisions by the field's width and height instead of seven
    // per lane: a lone wave issues an instruction every 5 to 8 cycles, and
    // the workgroup's first MFMA waits for its slowest wave); a lane then
    // fetches the pixels of its row blocks from the lanes that hold them.
    const uint32_t first = patchByteOf<kPixelUnits16>(a, span, span.m0 + lane);
    const uint32_t second =
        patchByteOf<kPixelUnits16>(a, span, span.m0 + 64 + lane);
#pragma unroll
    for (int i = 0; i != RB; ++i) {
      const int from = (16 * i + (lane & 15)) & 63;
      pixelByte[i] = uint32_t(__shfl(int(i < 4 ? first : second), from)) +
                     Mma::laneByte(lane >> 4);
    }
#pragma unroll
    for (int i = 0; i != RB; ++i)
      asm volatile("" ::"v"(pixelByte[i]));
  }, [&] {
#pragma unroll
    for (int u = kFirst; u != D; ++u)
      loadB(bf[u]);
  } MXK_STAMP_ARG);

  floatx4 acc[RB][2];
#pragma unroll
  for (int i = 0; i != RB; ++i)
#pragma unroll
    for (int c = 0; c != 2; ++c)
      acc[i][c] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

  // Own step j is k-step kt = 2 j + grp = slice * taps + tap; its A operands
  // sit at pixelByte + tapByte.  The offsets of 64 own steps at a time are
  // kept one per lane: lane l holds own step tableBase + 1 + l's, with bit 31
  // set on the wave's first step in a slice (tap 0 or 1).
  uint32_t tapTable = 0, tableBase = 0;
  auto fillTable = [&] {
    const uint32_t kt = 2 * (tableBase + 1 + lane) + grp;
    const uint32_t slice = a.divTaps(kt), tap = kt - slice * a.taps;
    const uint32_t kh = a.divKW(tap), kw = tap - kh * a.kW;
    tapTable = (slice * a.sliceBytes + kh * a.tapRowBytes +
                kw * a.tapColBytes) |
               (tap < 2 ? 0x80000000u : 0u);
  };
  fillTable();
  // (own step 0 is tap `grp` of slice 0)
  uint32_t tapByte;
  {
    const uint32_t kh = a.divKW(uint32_t(grp)), kw = uint32_t(grp) - kh * a.kW;
    tapByte = kh * a.tapRowBytes + kw * a.tapColBytes;
  }
  struct Operands {
    uintx4 x[RB][kReads];
  };
  auto readA = [&](Operands &o, uint32_t at) {
#pragma unroll
    for (int i = 0; i != RB; ++i)
#pragma unroll
      for (int r = 0; r != kReads; ++r)
        o.x[i][r] = *reinterpret_cast<const uintx4 *>(lds + pixelByte[i] + at +
                                                      64 * r);
  };
  auto multiply = [&](const uintx4(&b)[2][kReads], const Operands &o) {
#pragma unroll
    for (int i = 0; i != RB; ++i)
#pragma unroll
      for (int c = 0; c != 2; ++c)
        Mma::template mul<FA, FB>(b[c], o.x[i], acc[i][c]);
  };
  // MFMAs and the LDS reads of the next unit in turn (a wave issues in order
  // and an MFMA behind another waits for the pipe: what stands between two
  // of them costs nothing).
  auto interleave = [&] {
    __builtin_amdgcn_sched_group_barrier(0x002, RB, 0);
#pragma unroll
    for (int k = 0; k != RB * kReads; ++k) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2 / kReads, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
  };
  // One own step: kUnits units of MFMAs; `first` holds unit 0's operands and
  // gets the next step's on the way out when the step has two units, else
  // `second` does.  GUARD: the steps behind the last whole group of D.
  auto step = [&](auto guard, uintx4(&b)[kUnits][2][kReads], Operands &first,
                  Operands &second, uint32_t j) {
    constexpr bool GUARD = decltype(guard)::value;
    const bool more = !GUARD || j + 1 < own;
    uint32_t nextTap = 0;
    if (more) {
      const uint32_t entry = __builtin_amdgcn_readlane(tapTable, j - tableBase);
      nextTap = entry & 0x7fffffffu;
      if (entry & 0x80000000u) {
        // A new slice: its loads were issued before the loop, so they are
        // older than the weight loads of the last D steps (loads complete in
        // order); the barrier tells that the other waves' have landed too.
        if (j >= uint32_t(D))
          MXK_WAIT_VMCNT(4 * (D - 1));
        else
          MXK_WAIT_VMCNT(0);
        __builtin_amdgcn_s_barrier();
      }
    }
    if constexpr (!GUARD) {
      if constexpr (kUnits == 2) {
        readA(second, tapByte + 64);
        multiply(b[0], first);
        interleave();
        readA(first, nextTap);
        multiply(b[1], second);
        interleave();
      } else {
        readA(second, nextTap);
        multiply(b[0], first);
        interleave();
      }
      loadB(b);
      __builtin_amdgcn_sched_group_barrier(0x020, 4, 0);
    } else {
      if (j < own) {
        if constexpr (kUnits == 2) {
          readA(second, tapByte + 64);
          multiply(b[0], first);
          if (more)
            readA(first, nextTap);
          multiply(b[1], second);
        } else {
          if (more)
            readA(second, nextTap);
          multiply(b[0], first);
        }
      }
    }
    tapByte = nextTap;
  };
  Operands even, odd;
  // (nothing but these LDS reads pending at the head of the loop, so that
  // the waits inside it count reads)
  MXK_WAIT_LGKMCNT0();
  readA(even, tapByte);
  MXK_STAMP(6); // the other slices and weights requested: the k loop begins
  uint32_t j = 0;
  auto group = [&](auto guard) {
    if (j - tableBase == 64) {
      tableBase = j;
      fillTable();
    }
#pragma unroll
    for (int u = 0; u != D; u += 2) {
      if constexpr (kUnits == 2) {
        step(guard, bf[u], even, odd, j + u);
        step(guard, bf[u + 1], even, odd, j + u + 1);
      } else {
        step(guard, bf[u], even, odd, j + u);
        step(guard, bf[u + 1], odd, even, j + u + 1);
      }
    }
  };
  // (every step of a whole group has a successor to fetch for: the last
  // steps, at least one, are left to the guarded group)
  for (; j + D < own; j += D)
    group(std::false_type{});
  group(std::true_type{});
  MXK_STAMP(7); // own k-steps done

  // Sum the two waves' halves of K: wave grp 0 finishes row blocks
  // [0, kKeep16), wave grp 1 the others; each hands the other its sums of the
  // blocks it does not finish, through LDS - beside the patch where there is
  // room, else in its place, once everybody is done with it.
  if (a.exchangeByte == 0)
    __syncthreads();
  {
    uintx4 *exchange = reinterpret_cast<uintx4 *>(lds + a.exchangeByte);
    constexpr int kOutRow = kPatchBN * int(sizeof(OutT)) + 16;
    constexpr int kSlot = kKeep16 * 2; // 1 KB vectors a wave may be handed
    char *tileOut = lds + a.tileByte;
    auto give = [&](auto half) {
      constexpr int G = decltype(half)::value;
      constexpr int kFrom = G == 0 ? kKeep16 : 0;
      constexpr int kTo = G == 0 ? RB : kKeep16;
#pragma unroll
      for (int i = kFrom; i != kTo; ++i)
#pragma unroll
        for (int c = 0; c != 2; ++c)
          exchange[((wn * 2 + (1 - G)) * kSlot + (i - kFrom) * 2 + c) * 64 +
                   lane] = __builtin_bit_cast(uintx4, acc[i][c]);
    };
    if (grp == 0)
      give(std::integral_constant<int, 0>{});
    else
      give(std::integral_constant<int, 1>{});
    __syncthreads();
    MXK_STAMP(8); // both halves' sums handed over
    // the lane's channels of the tile: nLane + 16 c + e, e < 4
    const uint32_t nLane = wn * 32 + (lane >> 4) * 4;
    char *laneOut = tileOut + (lane & 15) * kOutRow + nLane * sizeof(OutT);
    auto keep = [&](auto half, auto biased) {
      constexpr int G = decltype(half)::value;
      constexpr int kFrom = G == 0 ? 0 : kKeep16;
      constexpr int kTo = G == 0 ? kKeep16 : RB;
      float bv[2][4] = {};
      if constexpr (decltype(biased)::value) {
        // (the channel count is a multiple of the output vector, so a run of
        // four channels is inside it or outside)
#pragma unroll
        for (int c = 0; c != 2; ++c) {
          const uint32_t n = nTile * kPatchBN + nLane + 16 * c;
          const OutT *b = bias + g * a.outChansPerGroup +
                          (n < a.outChansPerGroup ? n : 0);
          if constexpr (sizeof(OutT) == 2) {
            const uint2 raw = *reinterpret_cast<const uint2 *>(b);
            const __half2 lo = __builtin_bit_cast(__half2, raw.x),
                          hi = __builtin_bit_cast(__half2, raw.y);
            bv[c][0] = __low2float(lo), bv[c][1] = __high2float(lo);
            bv[c][2] = __low2float(hi), bv[c][3] = __high2float(hi);
          } else {
            const float4 raw = *reinterpret_cast<const float4 *>(b);
            bv[c][0] = raw.x, bv[c][1] = raw.y, bv[c][2] = raw.z,
            bv[c][3] = raw.w;
          }
        }
      }
      floatx4 other[kTo - kFrom][2];
#pragma unroll
      for (int i = kFrom; i != kTo; ++i)
#pragma unroll
        for (int c = 0; c != 2; ++c)
          other[i - kFrom][c] = __builtin_bit_cast(
              floatx4,
              exchange[((wn * 2 + G) * kSlot + (i - kFrom) * 2 + c) * 64 +
                       lane]);
#pragma unroll
      for (int i = kFrom; i != kTo; ++i)
#pragma unroll
        for (int c = 0; c != 2; ++c) {
          float v[4];
#pragma unroll
          for (int e = 0; e != 4; ++e) {
            v[e] = acc[i][c][e] + other[i - kFrom][c][e];
            if constexpr (EB == 1)
              v[e] *= scale;
            if constexpr (decltype(biased)::value)
              v[e] += bv[c][e];
          }
          storeOut4(reinterpret_cast<OutT *>(laneOut + i * 16 * kOutRow) +
                        16 * c,
                    v);
        }
    };
    if (bias) {
      if (grp == 0)
        keep(std::integral_constant<int, 0>{}, std::true_type{});
      else
        keep(std::integral_constant<int, 1>{}, std::true_type{});
    } else {
      if (grp == 0)
        keep(std::integral_constant<int, 0>{}, std::false_type{});
      else
        keep(std::integral_constant<int, 1>{}, std::false_type{});
    }
    __syncthreads();
    MXK_STAMP(9); // the tile is in LDS
    storeTile<128>(a, tileOut, out, t, g, nTile, span);
  }
#ifdef MXK_PATCH_STAMPS
  MXK_STAMP(10); // stores issued
  __builtin_amdgcn_s_waitcnt(0);
  MXK_STAMP(11); // ... and landed
  MXK_STAMP_REAL(15);
  stamps_[12] = own;
  if (patchStampSink && (t == 0 || t == kPatchThreads / 2)) {
    uint64_t *to = patchStampSink +
                   (size_t(blockIdx.x) * 2 + (t != 0)) * kStampSlots;
    for (int i = 0; i != kStampSlots; ++i)
      to[i] = stamps_[i];
  }
#endif
}

/// One element of the packed weights per thread:
/// [group][block of kTN x 32 channels][k-step][K half][32 channels][operand j]
/// [lane][16 bytes], or igemmPatch16Kernel's order of the same 4 KB per step
/// and 32 channels.
template <class T>
__global__ __launch_bounds__(256) void packPatchWeightsKernel(
    const T *__restrict__ src, T *__restrict__ dst, uint32_t co, uint32_t ci,
    uint32_t taps, uint32_t blocks, uint32_t kSteps, uint32_t packedTaps,
    uint64_t total, bool chansTransposed, bool selected,
    IgemmTapSelection select, bool blocks16) {
  constexpr uint32_t kVec = 16 / sizeof(T), kSlice = 128 / sizeof(T);
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  const uint32_t e = uint32_t(tid % kVec);
  const uint32_t lane = uint32_t(tid / kVec % 64);
  const uint32_t j = uint32_t(tid / (kVec * 64) % 2);
  const uint32_t c32 = uint32_t(tid / (kVec * 128) % kTN);
  const uint32_t half = uint32_t(tid / (kVec * 128 * kTN) % 2);
  const uint64_t rest = tid / (kVec * 256 * kTN);
  const uint32_t kt = uint32_t(rest % kSteps);
  const uint32_t block =
      uint32_t(rest / kSteps % (blocks / kTN)) * kTN + c32;
  const uint64_t g = rest / kSteps / (blocks / kTN);
  uint32_t n, within;
  if (blocks16) {
    // igemmPatch16Kernel: operand `half * 2 + j` of the step is (K unit,
    // column block) for fp16 and (column block, half of the lane's 32 bytes)
    // for fp8; lane = (K quarter, channel of the column block)
    const uint32_t quarter = lane >> 4;
    n = block * 32 + (sizeof(T) == 2 ? j : half) * 16 + (lane & 15);
    within = sizeof(T) == 2 ? half * 32 + quarter * 8 + e
                            : j * 64 + quarter * 16 + e;
  } else {
    const uint32_t h = lane >> 5;
    n = block * 32 + (lane & 31);
    within = sizeof(T) == 2 ? half * 32 + j * 16 + h * 8 + e
                            : half * 64 + h * 32 + j * 16 + e;
  }
  const uint32_t slice = kt / packedTaps;
  uint32_t tap = kt % packedTaps;
  const uint32_t c = slice * kSlice + within;
  T v = T(0);
  if (n < co && c < ci) {
    if (selected) {
      const uint32_t jw = tap % select.countW, r = tap / select.countW;
      const uint32_t i = r % select.countH, plane = r / select.countH;
      tap = ((select.firstD + plane * select.stepD) * select.kH +
             select.firstH + i * select.stepH) *
                select.kW +
            select.firstW + jw * select.stepW;
    }
    v = chansTransposed ? src[((g * ci + c) * co + n) * taps + tap]
                        : src[((g * co + n) * ci + c) * taps + tap];
  }
  dst[tid] = v;
}

uint32_t elemBytesOf(int type) {
  return type == kFloat ? 4 : type == kHalf ? 2 : 1;
}

/// Patch rows a tile of `blockM` consecutive output pixels can span.
uint32_t maxPatchRows(const IgemmDesc &d) {
  const uint64_t halo = uint64_t(d.kH - 1) * d.dilH;
  const uint64_t perImage = d.outH + halo;
  const uint64_t M = uint64_t(d.batch) * d.outH * d.outW;
  uint64_t most = 0;
  auto rowOf = [&](uint64_t m) {
    const uint64_t q = m / d.outW;
    return q / d.outH * perImage + q % d.outH;
  };
  const uint64_t tiles = (M + d.blockM - 1) / d.blockM;
  if (tiles <= 1u << 16) {
    for (uint64_t tile = 0; tile != tiles; ++tile) {
      const uint64_t m0 = tile * d.blockM;
      const uint64_t mL = std::min<uint64_t>(m0 + d.blockM, M) - 1;
      most = std::max(most, rowOf(mL) + halo + 1 - rowOf(m0));
    }
    return uint32_t(most);
  }
  const uint64_t outRows = (d.blockM - 1) / d.outW + 2;
  const uint64_t crossed =
      (d.blockM - 1) / (uint64_t(d.outH) * d.outW) + 1;
  return uint32_t(outRows - 1 + crossed * halo + halo + 1);
}

struct PatchShape {
  uint32_t eb, slices, taps, kSteps, rowLoads, rowPitch, maxRows, ldsBytes, rb;
  uint32_t exchangeByte, tileByte;
};

bool patchShape(const IgemmDesc &d, int inType, int outType, PatchShape &s) {
  if ((inType != kHalf && inType != kQuarter) ||
      (outType != kHalf && outType != kFloat))
    return false;
  s.eb = elemBytesOf(inType);
  if (d.inD != 1 || d.outD != 1 || d.kD != 1 || d.strideH != 1 ||
      d.strideW != 1 || d.inDilH != 1 || d.inDilW != 1 || d.outFullH != 0 ||
      d.outFullW != 0 || d.outTransposed || d.noTaps || d.splitK != 1)
    return false;
  const bool blocks16 = d.patch == 2;
  if (blocks16 ? d.blockM == 0 || d.blockM > uint32_t(kRows16) ||
                     uint64_t(d.kH) * d.kW < 2 || kTN != 1
               : d.blockM != 128 && d.blockM != 64)
    return false;
  s.rb = blocks16 ? 0 : d.blockM / 32;
  const uint64_t M = uint64_t(d.batch) * d.outH * d.outW;
  if (M == 0 || M > 0x7fffffffull || d.kH == 0 || d.kW == 0 ||
      d.inChansPerGroup == 0)
    return false;
  if ((d.inChansPerGroup * s.eb) % 128 != 0)
    return false;
  const uint32_t outVec = outType == kHalf ? 8 : 4;
  if (d.outChansPerGroup % outVec != 0)
    return false;
  s.slices = d.inChansPerGroup * s.eb / 128;
  s.taps = d.kH * d.kW;
  s.kSteps = s.slices * s.taps;
  const uint64_t cols = uint64_t(d.outW) + uint64_t(d.kW - 1) * d.dilW;
  const uint64_t units = blocks16 ? kPixelUnits16 : kPixelUnits;
  s.rowLoads = uint32_t((cols * units + 63) / 64);
  // The pitch from pixel to pixel spreads the 16-byte reads of an MFMA
  // operand over all 64 banks; the pitch of the rows continues that
  // progression (modulo the 256 bytes of the banks) from the last pixel of an
  // output row to the first of the next.
  const uint64_t pitch =
      uint64_t(d.outW) * 16 * units +
      ((cols - d.outW) * 16 * units + 255) / 256 * 256;
  s.maxRows = d.patchMaxRows ? d.patchMaxRows : maxPatchRows(d);
  // (a lane per patch row works out where the rows start)
  if (s.maxRows > 64)
    return false;
  const uint64_t patch = uint64_t(s.slices) * s.maxRows * pitch;
  if (patch > uint64_t(kLdsLimit))
    return false;
  s.rowPitch = uint32_t(pitch);
  const uint64_t exchange =
      blocks16 ? uint64_t(kPatchWaves) * kKeep16 * 2 * 1024
               : uint64_t(kPatchWaves) * (s.rb / 2) * kTN * 4 * 1024;
  const uint64_t tile = (blocks16 ? 128 : 32 * s.rb) *
                        (kPatchBN * (outType == kHalf ? 2 : 4) + 16);
  const uint64_t patchEnd = (patch + 1023) / 1024 * 1024;
  // Beside the patch where there is room (the waves then hand over their
  // sums as they finish, without waiting for the others to leave the patch);
  // the output tile, written once all have, goes over the patch if it ends
  // before the exchange area, else behind that.
  uint64_t bytes;
  if (patchEnd + exchange <= uint64_t(kLdsLimit) &&
      (tile <= patchEnd ||
       patchEnd + exchange + tile <= uint64_t(kLdsLimit))) {
    s.exchangeByte = uint32_t(patchEnd);
    s.tileByte = tile <= patchEnd ? 0 : uint32_t(patchEnd + exchange);
    bytes = patchEnd + exchange + (tile <= patchEnd ? 0 : tile);
  } else {
    s.exchangeByte = 0, s.tileByte = uint32_t(exchange);
    bytes = std::max(patch, exchange + tile);
  }
  if (bytes > uint64_t(kLdsLimit))
    return false;
  s.ldsBytes = uint32_t(bytes);
  const uint64_t wBytes = uint64_t(d.groups) *
                          ((d.outChansPerGroup + 127) / 128) * 4 * s.kSteps *
                          4096;
  // 32-bit offsets below kInvalid from the first image a tile reads
  const uint64_t imageBytes = uint64_t(d.inH) * d.inW * d.groups *
                              d.inChansPerGroup * s.eb;
  const uint64_t images = std::min<uint64_t>(
      d.batch, (d.blockM - 1) / (uint64_t(d.outH) * d.outW) + 2);
  if (wBytes >= kOutOfRange || images * imageBytes >= kInvalid)
    return false;
  // tiles and weight blocks are numbered in 32 bits
  const uint64_t tiles = (M + d.blockM - 1) / d.blockM *
                         ((d.outChansPerGroup + 127) / 128) * d.groups;
  return tiles <= 0x7fffffffull;
}

template <int EB, int FA, int FB, int RB, int D, class OutT>
hipError_t launchPatchKernel(const PatchArgs &a, uint32_t ldsBytes,
                             const void *in, const void *w, const void *bias,
                             void *out, float scale, hipStream_t stream) {
  auto kernel = &igemmPatchKernel<EB, FA, FB, RB, D, OutT>;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void *>(kernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
  if (attr != hipSuccess)
    return attr;
  const uint32_t blocks = a.mTiles * a.nTiles * a.groups;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kPatchThreads), ldsBytes,
                     stream, a, static_cast<const char *>(in),
                     static_cast<const char *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out),
                     scale);
  return hipGetLastError();
}

template <int EB, int FA, int FB, class OutT>
hipError_t dispatchPatchShape(const PatchShape &s, const PatchArgs &a,
                              const void *in, const void *w, const void *bias,
                              void *out, float scale, hipStream_t stream) {
  if (s.rb == 0) {
    auto kernel = &igemmPatch16Kernel<EB, FA, FB, kAhead16, OutT>;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void *>(kernel),
        hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
    if (attr != hipSuccess)
      return attr;
    hipLaunchKernelGGL(kernel, dim3(a.mTiles * a.nTiles * a.groups),
                       dim3(kPatchThreads), s.ldsBytes, stream, a,
                       static_cast<const char *>(in),
                       static_cast<const char *>(w),
                       static_cast<const OutT *>(bias),
                       static_cast<OutT *>(out), scale);
    return hipGetLastError();
  }
  if (s.rb == 4)
    return launchPatchKernel<EB, FA, FB, 4, 4, OutT>(a, s.ldsBytes, in, w,
                                                     bias, out, scale, stream);
  return launchPatchKernel<EB, FA, FB, 2, 4, OutT>(a, s.ldsBytes, in, w, bias,
                                                   out, scale, stream);
}

template <int EB, int FA, int FB>
hipError_t dispatchPatchOut(int outType, const PatchShape &s,
                            const PatchArgs &a, const void *in, const void *w,
                            const void *bias, void *out, float scale,
                            hipStream_t stream) {
  if (outType == kHalf)
    return dispatchPatchShape<EB, FA, FB, __half>(s, a, in, w, bias, out,
                                                  scale, stream);
  return dispatchPatchShape<EB, FA, FB, float>(s, a, in, w, bias, out, scale,
                                               stream);
}

} // namespace

uint32_t igemmPatchMaxRows(const IgemmDesc &d) { return maxPatchRows(d); }

bool igemmPatchTakes(const IgemmDesc &d, int inType, int outType) {
  PatchShape s;
  return patchShape(d, inType, outType, s);
}

uint64_t igemmPatchPackedElems(const IgemmDesc &d, int inType) {
  const uint32_t eb = elemBytesOf(inType);
  const uint64_t kSteps =
      uint64_t(d.inChansPerGroup) * eb / 128 * d.kH * d.kW;
  return uint64_t(d.groups) * ((d.outChansPerGroup + 127) / 128) * 4 * kSteps *
         (4096 / eb);
}

hipError_t launchPackIgemmPatchWeights(const IgemmDesc &d, int inType,
                                       const void *src, void *dst,
                                       uint32_t sourceTaps,
                                       hipStream_t stream,
                                       bool chansTransposed,
                                       const IgemmTapSelection *select) {
  const uint32_t eb = elemBytesOf(inType);
  if (eb == 4 || (d.inChansPerGroup * eb) % 128 != 0)
    return hipErrorInvalidValue;
  const uint64_t total = igemmPatchPackedElems(d, inType);
  if (total == 0)
    return hipSuccess;
  const uint32_t packedTaps = d.kH * d.kW;
  const uint32_t kSteps = d.inChansPerGroup * eb / 128 * packedTaps;
  const uint32_t blocks32 = (d.outChansPerGroup + 127) / 128 * 4;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const IgemmTapSelection chosen = select ? *select : IgemmTapSelection{};
  if (eb == 2)
    hipLaunchKernelGGL(packPatchWeightsKernel<uint16_t>, dim3(uint32_t(blocks)),
                       dim3(256), 0, stream,
                       static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst), d.outChansPerGroup,
                       d.inChansPerGroup, sourceTaps, blocks32, kSteps,
                       packedTaps, total, chansTransposed, select != nullptr,
                       chosen, d.patch == 2);
  else
    hipLaunchKernelGGL(packPatchWeightsKernel<uint8_t>, dim3(uint32_t(blocks)),
                       dim3(256), 0, stream, static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst), d.outChansPerGroup,
                       d.inChansPerGroup, sourceTaps, blocks32, kSteps,
                       packedTaps, total, chansTransposed, select != nullptr,
                       chosen, d.patch == 2);
  return hipGetLastError();
}

hipError_t launchIgemmPatch(const IgemmDesc &d, int inType, int outType,
                            const void *in, const void *weightsPacked,
                            const void *bias, void *out, const QuarterInfo &q,
                            hipStream_t stream) {
  PatchShape s;
  if (!patchShape(d, inType, outType, s))
    return hipErrorInvalidValue;
  PatchArgs a{};
  a.M = d.batch * d.outH * d.outW;
  a.tileM = d.blockM;
  a.mTiles = (a.M + d.blockM - 1) / d.blockM;
  a.nTiles = (d.outChansPerGroup + 127) / 128;
  a.groups = d.groups;
  a.outW = d.outW, a.outH = d.outH;
  a.rowsPerImage = d.outH + (d.kH - 1) * d.dilH;
  a.inH = d.inH;
  a.padH = d.padH, a.padW = d.padW;
  a.loH = d.loH, a.spanH = d.hiH - d.loH;
  a.loW = d.loW, a.spanW = d.hiW - d.loW;
  a.kW = d.kW, a.taps = s.taps, a.slices = s.slices, a.kSteps = s.kSteps;
  a.rowLoads = s.rowLoads;
  a.rowPitch = s.rowPitch;
  a.tapRowBytes = d.dilH * s.rowPitch;
  const uint32_t units = d.patch == 2 ? kPixelUnits16 : kPixelUnits;
  a.tapColBytes = d.dilW * 16 * units;
  a.rowUnits = (d.outW + (d.kW - 1) * d.dilW) * units;
  a.sliceBytes = s.maxRows * s.rowPitch;
  a.exchangeByte = s.exchangeByte, a.tileByte = s.tileByte;
  a.pixelBytes = d.groups * d.inChansPerGroup * s.eb;
  a.ciBytes = d.inChansPerGroup * s.eb;
  a.inRowBytes = d.inW * a.pixelBytes;
  a.imageBytes = d.inH * a.inRowBytes;
  a.inBytes = uint64_t(d.batch) * a.imageBytes;
  a.outChans = d.groups * d.outChansPerGroup;
  a.outChansPerGroup = d.outChansPerGroup;
  a.wBytes = uint32_t(igemmPatchPackedElems(d, inType) * s.eb);
  a.divOutW = makeFastDiv(d.outW);
  a.divOutH = makeFastDiv(d.outH);
  a.divNTiles = makeFastDiv(a.nTiles);
  a.divMTiles = makeFastDiv(a.mTiles);
  a.divRowLoads = makeFastDiv(s.rowLoads);
  a.divTaps = makeFastDiv(s.taps);
  a.divKW = makeFastDiv(d.kW);
  a.divRowsPerImage = makeFastDiv(a.rowsPerImage);
  const float scale = inType == kQuarter ? q.scale : 1.0f;
  if (inType == kHalf)
    return dispatchPatchOut<2, 0, 0>(outType, s, a, in, weightsPacked, bias,
                                     out, scale, stream);
  const int fa = q.inFormat != kE4M3 ? 1 : 0;
  const int fb = q.weightFormat != kE4M3 ? 1 : 0;
  if (fa == 0 && fb == 0)
    return dispatchPatchOut<1, 0, 0>(outType, s, a, in, weightsPacked, bias,
                                     out, scale, stream);
  if (fa == 0 && fb == 1)
    return dispatchPatchOut<1, 0, 1>(outType, s, a, in, weightsPacked, bias,
                                     out, scale, stream);
  if (fa == 1 && fb == 0)
    return dispatchPatchOut<1, 1, 0>(outType, s, a, in, weightsPacked, bias,
                                     out, scale, stream);
  return dispatchPatchOut<1, 1, 1>(outType, s, a, in, weightsPacked, bias, out,
                                   scale, stream);
}

} // namespace mxk

#ifdef MXK_PATCH_STAMPS
/// Stamps build only: the device buffer the stamped kernel writes to
/// ([workgroups][2][16] of 8 bytes), or null to switch the stamps off.
extern "C" int mxk_patch_stamp_sink(void *deviceBuffer) {
  return int(hipMemcpyToSymbol(HIP_SYMBOL(mxk::patchStampSink), &deviceBuffer,
                               sizeof(deviceBuffer)));
}
#endif

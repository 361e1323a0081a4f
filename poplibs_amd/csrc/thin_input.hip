// Convolution of an input with very few channels (an image's three, a
// waveform's one) on the matrix cores, without padding the channels.
//
// In a channels-last image the kW pixels under one kernel row are kW * Ci
// neighbouring elements - 21 for a 7 x 7 kernel over RGB: a kernel row is
// ceil(kW * Ci / 8) chunks of 8 elements, and four chunks (of one kernel row
// or of neighbouring ones) make a k-step of 32.  K = 6 * 32 for that layer
// where padding the channels to a whole 16-byte vector gives 7 * 7 * 8 = 392
// and costs a copy of the input besides; a 3 x 3 kernel over RGB is two
// k-steps.  The price is alignment: a window starts at any even
// byte, so the operand is read from LDS as five aligned dwords and shifted
// into place.
//
//   workgroup  = 4 waves; one image's TH output rows at a time (persistent);
//                the input rows under them lie in LDS, zeros around them
//   wave       = blocks of 16 neighbouring output pixels, round robin
//   MFMA       = v_mfma_f32_16x16x32_f16, weights as the row operand:
//                D[co][pixel] += W[co][k] * X[k][pixel], one per k-step and
//                block of 16 output channels; all weights stay in registers
//   output     = output channels are dealt to the MFMA rows so that a lane
//                ends up with 4 * CB neighbouring channels of one pixel
#include "igemm_common.hpp"
#include "kernels.hpp"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

namespace mxk {
namespace {

constexpr int kThinThreads = 256;

struct ThinArgs {
  ThinInputDesc d;
  uint32_t tileRows;   // TH: output rows per tile
  uint32_t ldsRows;    // (TH - 1) * strideH + kH
  uint32_t pitch;      // bytes of an LDS row
  uint32_t dataOff;    // byte of input column 0 in an LDS row (16-aligned)
  uint32_t rowBytes;   // inW * ci * 2
  uint32_t tilesPerImage, tiles;
  uint32_t colBlocks;  // blocks of 16 output pixels per row
  FastDiv divTilesPerImage, divColBlocks;
  FastDiv divRowUnits; // by the 16-byte vectors (or dwords) of an input row
  FastDiv divBorder;   // by the dwords of zeros left and right of a row
  uint32_t biasByte;   // where the fp32 bias lies in LDS
  uint32_t weightByte; // ... and the packed weights, on their way to registers
  FastDiv divChunksPerRow; // by the chunks of 8 elements of a kernel row
  uint32_t cutElems;   // elements of a row in truncated columns
  FastDiv divCut;
};

/// First of the four neighbouring output channels that lane quarter Q holds
/// of channel block cb (MFMA rows 4 Q .. 4 Q + 3), of `blocks` blocks.  The
/// blocks go in pairs of 32 channels: within a pair quarter Q holds channels
/// 8 Q .. 8 Q + 7 (four from either block), so that a pixel's 64 bytes (fp16)
/// are written by one store instruction's four quarters, whole; an odd last
/// block stands alone with channels 4 Q .. 4 Q + 3.
__host__ __device__ inline uint32_t thinChannelBase(uint32_t cb, uint32_t Q,
                                                    uint32_t blocks) {
  const uint32_t pair = cb / 2;
  return (cb ^ 1u) < blocks ? pair * 32 + Q * 8 + (cb & 1u) * 4
                            : pair * 32 + Q * 4;
}

/// Output channel held by MFMA row m of channel block cb.
__host__ __device__ inline uint32_t thinChannelOf(uint32_t cb, uint32_t m,
                                                  uint32_t blocks) {
  return thinChannelBase(cb, m / 4, blocks) + m % 4;
}

/// Chunks of 8 elements per kernel row, in all, and the k-steps they make.
__host__ __device__ inline uint32_t thinChunksPerRow(const ThinInputDesc &d) {
  return (d.kW * d.inChans + 7) / 8;
}
__host__ __device__ inline uint32_t thinChunks(const ThinInputDesc &d) {
  return d.kH * thinChunksPerRow(d);
}
__host__ __device__ inline uint32_t thinKSteps(const ThinInputDesc &d) {
  return (thinChunks(d) + 3) / 4;
}

/// Packed weights [cb][k-step][lane][8]: lane l holds MFMA row l % 16 and
/// chunk 4 * step + l / 16 - elements 8 * part .. + 7 of kernel row `row`,
/// chunk = row * chunksPerRow + part, element = kw * Ci + c - with zeros
/// beyond kW * Ci and beyond the last chunk.
__global__ void packThinWeightsKernel(const __half *__restrict__ src,
                                      __half *__restrict__ dst,
                                      ThinInputDesc d, uint32_t total) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total)
    return;
  const uint32_t steps = thinKSteps(d), perRow = thinChunksPerRow(d);
  const uint32_t e = i % 8, lane = (i / 8) % 64;
  const uint32_t step = (i / 512) % steps, cb = i / 512 / steps;
  const uint32_t chunk = 4 * step + lane / 16;
  const uint32_t kh = chunk / perRow, k = (chunk % perRow) * 8 + e;
  const uint32_t co = thinChannelOf(cb, lane % 16, d.outChans / 16);
  const uint32_t kw = k / d.inChans, c = k % d.inChans;
  __half v = __float2half(0.0f);
  if (kh < d.kH && kw < d.kW)
    v = src[((size_t(co) * d.inChans + c) * d.kH + kh) * d.kW + kw];
  dst[i] = v;
}

/// Input rows ih0 .. ih0 + ldsRows - 1 of an image into LDS in units of V
/// (16 or 4 bytes), zeros for rows outside [loH, hiH).
template <class V>
__device__ __forceinline__ void copyRows(const ThinArgs &a, char *lds,
                                         const char *img, int32_t ih0, int t) {
  constexpr int kBatch = 8;
  const uint32_t units = a.rowBytes / uint32_t(sizeof(V));
  const uint32_t total = a.ldsRows * units;
  for (uint32_t first = 0; first < total; first += kBatch * kThinThreads) {
    V v[kBatch];
    uint32_t at[kBatch];
#pragma unroll
    for (int u = 0; u != kBatch; ++u) {
      const uint32_t i = first + u * kThinThreads + t;
      const uint32_t row = a.divRowUnits(i), c = i - row * units;
      const int32_t ih = ih0 + int32_t(row);
      at[u] = i < total ? row * a.pitch + a.dataOff + c * uint32_t(sizeof(V))
                        : ~0u;
      v[u] = V{};
      if (i < total && ih >= int32_t(a.d.loH) && ih < int32_t(a.d.hiH))
        v[u] = reinterpret_cast<const V *>(img + size_t(ih) * a.rowBytes)[c];
    }
#pragma unroll
    for (int u = 0; u != kBatch; ++u)
      if (at[u] != ~0u)
        *reinterpret_cast<V *>(lds + at[u]) = v[u];
  }
}

template <int CB, int KS, class OutT>
__global__ __launch_bounds__(kThinThreads)
    __attribute__((amdgpu_waves_per_eu(2))) void thinInputKernel(
    ThinArgs a, const __half *__restrict__ in,
    const __half *__restrict__ weightsPacked, const OutT *__restrict__ bias,
    OutT *__restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const ThinInputDesc &d = a.d;
  const int t = threadIdx.x, lane = t & 63;
  // (the same for every lane of a wave, and said so: what depends on it and
  // the launch's constants alone - a block's row and column, the start of
  // its outputs - is then worked out on the scalar unit)
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);

  // The weights go through LDS into every wave's registers; their loads are
  // issued first and written to LDS behind the first tile's rows, so that
  // one trip to memory covers both.
  constexpr int kWeightVecs = CB * KS * 64;
  uintx4 weightVec[(kWeightVecs + kThinThreads - 1) / kThinThreads];
#pragma unroll
  for (int u = 0; u * kThinThreads < kWeightVecs; ++u)
    if (u * kThinThreads + t < kWeightVecs)
      weightVec[u] = reinterpret_cast<const uintx4 *>(
          weightsPacked)[u * kThinThreads + t];

  // Zeros left and right of the rows' data: written once, never overwritten.
  {
    const uint32_t left = a.dataOff / 4;
    const uint32_t right = (a.pitch - a.dataOff - a.rowBytes) / 4;
    const uint32_t per = left + right;
    for (uint32_t i = t; i < a.ldsRows * per; i += kThinThreads) {
      const uint32_t row = a.divBorder(i), c = i - row * per;
      const uint32_t byte =
          c < left ? c * 4 : a.dataOff + a.rowBytes + (c - left) * 4;
      *reinterpret_cast<uint32_t *>(lds + row * a.pitch + byte) = 0;
    }
  }

  // This lane's part of a k-step's operand: pixel lane % 16 of a block,
  // chunk 4 * step + lane / 16 - eight elements of one kernel row.  The
  // pixel's first byte within an LDS row, for block 0 (a block further on is
  // 16 * strideW pixels further on):
  const uint32_t pixelBytes = d.inChans * 2;
  const int32_t colByte0 =
      int32_t(a.dataOff) +
      (int32_t((lane & 15) * d.strideW) - d.padW) * int32_t(pixelBytes);
  // (a multiple of 32 bytes, like a chunk's 16 and the rows' pitch: every
  // operand of a lane starts at the same byte of a dword)
  const uint32_t blockStep = 16 * d.strideW * pixelBytes;
  const uint32_t shift = uint32_t(colByte0) & 3u;
  // Per k-step: where the lane's chunk lies from the block's first row (the
  // aligned dword at or below it), and the byte permute that turns the
  // aligned dwords i and i + 1 into the operand's dword i - selector byte
  // b + shift picks that byte of the pair, 0x0c a zero: for the elements
  // beyond the kernel row's kW * Ci (the next pixels') and for chunks beyond
  // the last.
  uint32_t chunkAt[KS], pick[KS][4];
  {
    const uint32_t perRow = thinChunksPerRow(d), chunks = thinChunks(d);
    const uint32_t kEnd = d.kW * d.inChans;
#pragma unroll
    for (int q = 0; q != KS; ++q) {
      const uint32_t chunk = 4 * q + (lane >> 4);
      const bool there = chunk < chunks;
      const uint32_t row = there ? a.divChunksPerRow(chunk) : 0;
      const uint32_t part = there ? chunk - row * perRow : 0;
      chunkAt[q] = (uint32_t(colByte0) & ~3u) + row * a.pitch + part * 16;
#pragma unroll
      for (int i = 0; i != 4; ++i) {
        const uint32_t k = part * 8 + 2 * i;
        const uint32_t lo =
            there && k < kEnd ? (shift | ((shift + 1) << 8)) : 0x0c0cu;
        const uint32_t hi = there && k + 1 < kEnd
                                ? ((shift + 2) | ((shift + 3) << 8))
                                : 0x0c0cu;
        pick[q][i] = lo | (hi << 16);
      }
    }
  }
  // the bias, as fp32, behind the rows in LDS: a lane's 4 * CB channels are
  // read back when a block is stored
  const uint32_t quarter = lane >> 4;
  float *biasLds = reinterpret_cast<float *>(lds + a.biasByte);
  if (t < CB * 16)
    biasLds[t] = bias ? Load<OutT>::at(bias, t, 0) : 0.0f;

  const bool vec16 = (a.rowBytes & 15) == 0;
  // Input rows of a tile into LDS, zeros for rows outside the image (loads in
  // batches of eight per thread, all on their way before the first is
  // written to LDS).
  auto stage = [&](uint32_t tile) {
    const uint32_t image = a.divTilesPerImage(tile);
    const uint32_t oh0 = (tile - image * a.tilesPerImage) * a.tileRows;
    const int32_t ih0 = int32_t(oh0 * d.strideH) - d.padH;
    const char *img = reinterpret_cast<const char *>(
        in + size_t(image) * d.inH * d.inW * d.inChans);
    if (vec16)
      copyRows<uintx4>(a, lds, img, ih0, t);
    else
      copyRows<uint32_t>(a, lds, img, ih0, t);
    if (a.cutElems) {
      // truncated columns read as zeros: wiped once the rows are in
      __syncthreads();
      const uint32_t left = d.loW * d.inChans;
      for (uint32_t i = t; i < a.ldsRows * a.cutElems; i += kThinThreads) {
        const uint32_t row = a.divCut(i), c = i - row * a.cutElems;
        const uint32_t elem = c < left ? c : d.hiW * d.inChans + (c - left);
        *reinterpret_cast<__half *>(lds + row * a.pitch + a.dataOff +
                                    elem * 2) = __float2half(0.0f);
      }
    }
  };
  if (blockIdx.x < a.tiles)
    stage(blockIdx.x);
  {
    uintx4 *dst = reinterpret_cast<uintx4 *>(lds + a.weightByte);
#pragma unroll
    for (int u = 0; u * kThinThreads < kWeightVecs; ++u)
      if (u * kThinThreads + t < kWeightVecs)
        dst[u * kThinThreads + t] = weightVec[u];
  }
  __syncthreads();
  half8 w[CB][KS];
#pragma unroll
  for (int cb = 0; cb != CB; ++cb)
#pragma unroll
    for (int q = 0; q != KS; ++q)
      w[cb][q] = reinterpret_cast<const half8 *>(
          lds + a.weightByte)[(cb * KS + q) * 64 + lane];

  for (uint32_t tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
    const uint32_t image = a.divTilesPerImage(tile);
    const uint32_t oh0 = (tile - image * a.tilesPerImage) * a.tileRows;
    if (tile != blockIdx.x) {
      stage(tile);
      __syncthreads();
    }

    const uint32_t rowsHere =
        a.tileRows < d.outH - oh0 ? a.tileRows : d.outH - oh0;
    const uint32_t blocks = rowsHere * a.colBlocks;
    constexpr uint32_t kWaves = kThinThreads / 64;
    for (uint32_t b = wave; b < blocks; b += kWaves) {
      const uint32_t r = a.divColBlocks(b), cbk = b - r * a.colBlocks;
      const char *base = lds + r * d.strideH * a.pitch + cbk * blockStep;
      // all of the block's reads, then its arithmetic
      uint32_t x[KS][5];
#pragma unroll
      for (int q = 0; q != KS; ++q)
#pragma unroll
        for (int i = 0; i != 5; ++i)
          x[q][i] = reinterpret_cast<const uint32_t *>(base + chunkAt[q])[i];
      // the sums start from the bias
      floatx4 acc[CB];
#pragma unroll
      for (int cb = 0; cb != CB; ++cb)
        acc[cb] = *reinterpret_cast<const floatx4 *>(
            biasLds + thinChannelBase(cb, quarter, CB));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int q = 0; q != KS; ++q) {
        uintx4 u;
        u.x = __builtin_amdgcn_perm(x[q][1], x[q][0], pick[q][0]);
        u.y = __builtin_amdgcn_perm(x[q][2], x[q][1], pick[q][1]);
        u.z = __builtin_amdgcn_perm(x[q][3], x[q][2], pick[q][2]);
        u.w = __builtin_amdgcn_perm(x[q][4], x[q][3], pick[q][3]);
        half8 xs;
        __builtin_memcpy(&xs, &u, 16);
#pragma unroll
        for (int cb = 0; cb != CB; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[cb][q], xs,
                                                           acc[cb], 0, 0, 0);
      }
      const uint32_t ow = cbk * 16 + (lane & 15);
      if (ow < d.outW) {
        OutT *dst = out + ((size_t(image) * d.outH + oh0 + r) * d.outW + ow) *
                              d.outChans;
        // a pair of channel blocks: eight neighbouring channels per lane
#pragma unroll
        for (int cb = 0; cb + 1 < CB; cb += 2) {
          OutT *at = dst + thinChannelBase(cb, quarter, CB);
          if constexpr (sizeof(OutT) == 2) {
            const __half2 h[4] = {
                roundPairToHalf(acc[cb][0], acc[cb][1]),
                roundPairToHalf(acc[cb][2], acc[cb][3]),
                roundPairToHalf(acc[cb + 1][0], acc[cb + 1][1]),
                roundPairToHalf(acc[cb + 1][2], acc[cb + 1][3])};
            uintx4 u;
            __builtin_memcpy(&u, h, 16);
            *reinterpret_cast<uintx4 *>(at) = u;
          } else {
            const float v0[4] = {acc[cb][0], acc[cb][1], acc[cb][2],
                                 acc[cb][3]};
            const float v1[4] = {acc[cb + 1][0], acc[cb + 1][1],
                                 acc[cb + 1][2], acc[cb + 1][3]};
            storeOut4(at, v0);
            storeOut4(at + 4, v1);
          }
        }
        if constexpr (CB % 2 == 1) {
          const float v[4] = {acc[CB - 1][0], acc[CB - 1][1], acc[CB - 1][2],
                              acc[CB - 1][3]};
          storeOut4(dst + thinChannelBase(CB - 1, quarter, CB), v);
        }
      }
    }
    __syncthreads();
  }
}

struct ThinShape {
  uint32_t kSteps; // k-steps of four chunks: 1 to 7
  uint32_t tileRows, ldsRows, pitch, dataOff, rowBytes, colBlocks;
  uint32_t ldsBytes;
  bool ok;
};

uint32_t alignUp(uint32_t v, uint32_t to) { return (v + to - 1) / to * to; }

ThinShape thinShape(const ThinInputDesc &d, uint32_t cus) {
  ThinShape s{};
  s.kSteps = thinKSteps(d);
  const uint32_t pixelBytes = d.inChans * 2;
  s.rowBytes = d.inW * pixelBytes;
  s.colBlocks = (d.outW + 15) / 16;
  const uint32_t padLeft = d.padW > 0 ? uint32_t(d.padW) : 0;
  s.dataOff = alignUp(padLeft * pixelBytes, 16);
  // the last lane of the last block reads 20 bytes from (at most) here
  const int64_t lastRead =
      int64_t(s.dataOff) +
      (int64_t(s.colBlocks * 16 - 1) * d.strideW - d.padW) * pixelBytes + 48 +
      24;
  const int64_t extent =
      std::max<int64_t>(lastRead, int64_t(s.dataOff) + s.rowBytes);
  if (extent > (1 << 16))
    return s;
  s.pitch = alignUp(uint32_t(extent), 16);
  const uint32_t weightBytes = (d.outChans / 16) * s.kSteps * 1024;
  // the largest tile of 16, 8, ... output rows that fits 64 KB and leaves
  // three tiles to two CUs; failing that the smallest
  uint32_t chosen = 0;
  for (uint32_t th = 16; th != 0; th /= 2) {
    const uint32_t rows = (th - 1) * d.strideH + d.kH;
    if (uint64_t(rows) * s.pitch > 64 * 1024)
      continue;
    chosen = th;
    if (uint64_t(d.batch) * ((d.outH + th - 1) / th) * 2 >= 3ull * cus)
      break;
  }
  if (!chosen)
    return s;
  s.tileRows = std::min(chosen, std::max(1u, d.outH));
  s.ldsRows = (s.tileRows - 1) * d.strideH + d.kH;
  // (+ 256 bytes behind them for the bias, then the weights)
  s.ldsBytes = s.ldsRows * s.pitch + 256 + weightBytes;
  s.ok = true;
  return s;
}

template <int CB, int KS, class OutT>
hipError_t launchOne(const ThinArgs &a, uint32_t grid, uint32_t ldsBytes,
                     const void *in, const void *w, const void *bias,
                     void *out, hipStream_t stream) {
  hipLaunchKernelGGL((thinInputKernel<CB, KS, OutT>), dim3(grid),
                     dim3(kThinThreads), ldsBytes, stream, a,
                     static_cast<const __half *>(in),
                     static_cast<const __half *>(w),
                     static_cast<const OutT *>(bias),
                     static_cast<OutT *>(out));
  return hipGetLastError();
}

template <int CB, class OutT>
hipError_t launchRows(uint32_t rows, const ThinArgs &a, uint32_t grid,
                      uint32_t ldsBytes, const void *in, const void *w,
                      const void *bias, void *out, hipStream_t stream) {
  switch (rows) {
#define MXK_THIN_CASE(n)                                                       \
  case n:                                                                      \
    return launchOne<CB, n, OutT>(a, grid, ldsBytes, in, w, bias, out, stream);
    MXK_THIN_CASE(1)
    MXK_THIN_CASE(2)
    MXK_THIN_CASE(3)
    MXK_THIN_CASE(4)
    MXK_THIN_CASE(5)
    MXK_THIN_CASE(6)
    MXK_THIN_CASE(7)
#undef MXK_THIN_CASE
  }
  return hipErrorInvalidValue;
}

template <class OutT>
hipError_t launchBlocks(uint32_t cb, uint32_t rows, const ThinArgs &a,
                        uint32_t grid, uint32_t ldsBytes, const void *in,
                        const void *w, const void *bias, void *out,
                        hipStream_t stream) {
  switch (cb) {
  case 1:
    return launchRows<1, OutT>(rows, a, grid, ldsBytes, in, w, bias, out,
                               stream);
  case 2:
    return launchRows<2, OutT>(rows, a, grid, ldsBytes, in, w, bias, out,
                               stream);
  case 3:
    return launchRows<3, OutT>(rows, a, grid, ldsBytes, in, w, bias, out,
                               stream);
  case 4:
    return launchRows<4, OutT>(rows, a, grid, ldsBytes, in, w, bias, out,
                               stream);
  }
  return hipErrorInvalidValue;
}

} // namespace

bool thinInputTakes(const ThinInputDesc &d, int inType, int outType) {
  if (inType != kHalf || (outType != kHalf && outType != kFloat))
    return false;
  if (d.batch == 0 || d.outH == 0 || d.outW == 0 || d.inH == 0 || d.inW == 0)
    return false;
  if (d.loH > d.hiH || d.hiH > d.inH || d.loW > d.hiW || d.hiW > d.inW)
    return false;
  if (d.inChans == 0 || d.inChans > 4 || d.kW * d.inChans > 32 ||
      d.kH == 0 || d.kH > 28 || d.kH * d.kW < 2)
    return false;
  // 7 k-steps of four 8-element chunks at most (the weights' registers)
  if (thinChunks(d) > 28)
    return false;
  if (d.outChans % 16 != 0 || d.outChans > 64)
    return false;
  // rows are copied in dwords
  if ((d.inW * d.inChans) % 2 != 0)
    return false;
  if (d.strideH == 0 || d.strideW == 0 || d.strideW > 64 ||
      d.padW > 4096 || d.padW < -4096 || d.padH > (1 << 20) ||
      d.padH < -(1 << 20))
    return false;
  // every window inside the (padded) rows kept in LDS: nothing is read
  // left of the row's start
  if (d.padW < 0)
    return false;
  if (uint64_t(d.batch) * d.outH * d.outW * d.outChans >= (1ull << 32) ||
      uint64_t(d.batch) * d.inH * d.inW * d.inChans >= (1ull << 32))
    return false;
  return thinShape(d, 256).ok;
}

uint64_t thinInputPackedElems(const ThinInputDesc &d) {
  return uint64_t(d.outChans / 16) * thinKSteps(d) * 512;
}

uint32_t thinInputKSteps(const ThinInputDesc &d) { return thinKSteps(d); }

ThinInputLaunch thinInputLaunchShape(const ThinInputDesc &d, uint32_t cus) {
  const ThinShape s = thinShape(d, cus);
  ThinInputLaunch l{};
  l.tileRows = s.tileRows;
  l.ldsBytes = s.ldsBytes;
  const uint64_t tiles =
      uint64_t(d.batch) * ((d.outH + s.tileRows - 1) / std::max(1u, s.tileRows));
  // (two workgroups to a CU: what the registers of the largest variant -
  // 64 output channels, 7 kernel rows - allow)
  l.workgroups = std::min<uint64_t>(tiles, uint64_t(cus) * 2);
  l.tiles = tiles;
  return l;
}

hipError_t launchPackThinInputWeights(const ThinInputDesc &d, const void *src,
                                      void *dst, hipStream_t stream) {
  const uint32_t total = uint32_t(thinInputPackedElems(d));
  hipLaunchKernelGGL(packThinWeightsKernel, dim3((total + 255) / 256),
                     dim3(256), 0, stream, static_cast<const __half *>(src),
                     static_cast<__half *>(dst), d, total);
  return hipGetLastError();
}

hipError_t launchThinInput(const ThinInputDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, hipStream_t stream) {
  if (!thinInputTakes(d, inType, outType))
    return hipErrorInvalidValue;
  const ThinShape s = thinShape(d, 256);
  const ThinInputLaunch l = thinInputLaunchShape(d, 256);
  ThinArgs a{};
  a.d = d;
  a.tileRows = s.tileRows, a.ldsRows = s.ldsRows, a.pitch = s.pitch;
  a.dataOff = s.dataOff, a.rowBytes = s.rowBytes;
  a.tilesPerImage = (d.outH + s.tileRows - 1) / s.tileRows;
  a.tiles = uint32_t(l.tiles);
  a.colBlocks = s.colBlocks;
  a.divTilesPerImage = makeFastDiv(a.tilesPerImage);
  a.divColBlocks = makeFastDiv(a.colBlocks);
  a.divRowUnits =
      makeFastDiv((s.rowBytes & 15) == 0 ? s.rowBytes / 16 : s.rowBytes / 4);
  a.divBorder = makeFastDiv((s.pitch - s.rowBytes) / 4);
  a.biasByte = s.ldsRows * s.pitch;
  a.weightByte = a.biasByte + 256;
  a.divChunksPerRow = makeFastDiv(thinChunksPerRow(d));
  a.cutElems = (d.loW + (d.inW - d.hiW)) * d.inChans;
  a.divCut = makeFastDiv(a.cutElems);
  if (l.tiles >= (1ull << 31))
    return hipErrorInvalidConfiguration;
  const uint32_t grid = uint32_t(l.workgroups);
  if (outType == kHalf)
    return launchBlocks<__half>(d.outChans / 16, s.kSteps, a, grid,
                                s.ldsBytes, in, weightsPacked, bias, out,
                                stream);
  return launchBlocks<float>(d.outChans / 16, s.kSteps, a, grid,
                             s.ldsBytes, in, weightsPacked, bias, out, stream);
}

} // namespace mxk

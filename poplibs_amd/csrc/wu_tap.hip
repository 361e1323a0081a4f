// Weight deltas of a dense layer (any stride) on the matrix cores, straight
// from the layer's own tensors:
//   dW[g][co][ci][kh][kw] = sum over b, y, x of
//       deltas[b][y][x][g][co] *
//           acts[b][y strideH + kh - padH][x strideW + kw - padW][g][ci]
// (PopLibs runs this as a convolution of its own with batch and channels
// exchanged, lib/poplin/Convolution.cpp:3437-3483 calculateWeightDeltas, whose
// tensors Poplar rearranges on the exchange; here that would be two transposes
// through HBM per pass.)
//
// As a matrix product per kernel tap: M = output channels, N = input channels,
// K = pixels (b, y, x).  Both operands are stored with K outermost - a pixel's
// channels are consecutive, the next pixel follows - which is the wrong way
// round for an MFMA (a lane holds 8 consecutive k of one row).  gfx950's
// transposing LDS read (ds_read_b64_tr_b16) turns that round on the way to the
// registers: 16 lanes that point at 4 k-rows of 16 consecutive channels get,
// each, one channel's 4 k values.  So the tensors go from HBM to LDS as they
// are, 1 KB per wave-wide load, and no transposed copy is ever made.
//
// Workgroup = (chunk of pixels, tap, 128 x 128 tile of channels), 8 waves.
// The pixels of a chunk pass through LDS in super-steps of 64: two 32-pixel
// halves, each half a tile of deltas [32][128 co] and one of activations
// [32][128 ci] (the tap's shifted view of the input: pixel + tap offset, zeros
// outside - out-of-range buffer offsets).  Waves 0-3 multiply the first half,
// waves 4-7 the second: a 2 x 2 grid of 64 x 64 tiles per half, the two waves
// of a SIMD covering each other's latencies; their sums meet in LDS at the
// end.  The fp32 tile goes to the workspace; a second kernel adds the chunks'
// tiles in a fixed order and writes the deltas in weight order.
//
// LDS tile: 32 rows (pixels) of 256 bytes, no padding (a wave-wide load
// writes 4 rows at once); the 16-byte chunk c of row r sits at chunk position
// c ^ 2 ((r % 4) + 4 ((r / 8) % 2)), which spreads the 16 rows a transposing
// read touches over all banks.
#include "igemm_common.hpp"

#include <algorithm>

namespace mxk {
namespace {

constexpr int kWuThreads = 512;
constexpr int kWuStages = 4;
constexpr int kWuTileBytes = 32 * 256;           // 32 pixels x 128 channels
constexpr int kWuStageBytes = 4 * kWuTileBytes;   // 2 halves x 2 operands
constexpr int kWuOutRow = 128 * 4 + 16;           // fp32 tile row in LDS
constexpr uint32_t kWuInvalid = 0x40000000u;

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4 *LdsShortx4;

struct WuTapArgs {
  WuTapDesc d;
  uint32_t M;              // pixels: batch * outH * outW
  uint32_t taps, ciTiles, coTiles;
  uint32_t chunks, tilesPerChunk;
  uint32_t actPixelBytes, deltaPixelBytes; // groups * channels * 2
  uint32_t actImageBytes;                  // inH * inW * actPixelBytes
  uint32_t stepX, stepY, stepImages;       // 64 pixels as columns, rows, images
  uint64_t actBytes, deltaBytes;
  FastDiv divOutW, divOutH, divTaps, divCiTiles, divCoTiles, divKW;
  FastDiv divTilesPerChunk;
};

__device__ __forceinline__ half8 transposedOperand(const char *at) {
#if defined(__HIP_DEVICE_COMPILE__)
  // rows r .. r + 3 and r + 4 .. r + 7 of the lane's 16 channels
  const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (LdsShortx4)(at));
  const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (LdsShortx4)(at + 4 * 256));
  typedef short shortx8 __attribute__((ext_vector_type(8)));
  const shortx8 both = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  return __builtin_bit_cast(half8, both);
#else
  return half8{};
#endif
}

__global__ __launch_bounds__(kWuThreads) void wuTapKernel(
    const WuTapArgs a, const char *__restrict__ acts,
    const char *__restrict__ deltas, float *__restrict__ partial) {
  extern __shared__ __align__(16) char lds[];
  const WuTapDesc &d = a.d;
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int grp = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;

  // workgroup -> (chunk, group, tap, ci tile, co tile), co tile fastest
  const uint32_t chunk = a.divTilesPerChunk(blockIdx.x);
  uint32_t id = blockIdx.x - chunk * a.tilesPerChunk;
  uint32_t q = a.divCoTiles(id);
  const uint32_t coTile = id - q * a.coTiles;
  id = q, q = a.divCiTiles(id);
  const uint32_t ciTile = id - q * a.ciTiles;
  id = q, q = a.divTaps(id);
  const uint32_t tap = id - q * a.taps;
  const uint32_t g = q;
  const uint32_t kh = a.divKW(tap), kw = tap - kh * d.kW;
  const uint32_t p0 = chunk * d.chunkPixels;
  const uint32_t p1 = p0 + d.chunkPixels < a.M ? p0 + d.chunkPixels : a.M;
  const uint32_t steps = (p1 - p0 + 63) >> 6;

  // Loads.  Wave w brings rows 4 w .. 4 w + 3 of every tile: lane l row
  // 4 w + l / 16, chunk position l % 16, which holds channel chunk
  // (l % 16) ^ swizzle(row).
  const uint32_t row = wave * 4 + (lane >> 4);
  const uint32_t chanChunk =
      (lane & 15) ^ (2 * ((row & 3) + 4 * ((row >> 3) & 1)));
  const __amdgpu_buffer_rsrc_t actBuf = bufferOf(
      acts, uint32_t(a.actBytes < kWuInvalid ? a.actBytes : kWuInvalid));
  const __amdgpu_buffer_rsrc_t deltaBuf = bufferOf(
      deltas, uint32_t(a.deltaBytes < kWuInvalid ? a.deltaBytes : kWuInvalid));
  const uint32_t actChan = ciTile * 128 + chanChunk * 8;
  const uint32_t deltaChan = coTile * 128 + chanChunk * 8;
  const uint32_t actLane = actChan < d.ci ? (g * d.ci + actChan) * 2 : kWuInvalid;
  const uint32_t deltaLane =
      deltaChan < d.co ? (g * d.co + deltaChan) * 2 : kWuInvalid;
  // Steps are loaded in order, so each lane keeps where its two pixels of the
  // next step are (column, row, image) and moves them on by 64 pixels with
  // two carries instead of taking the pixel number apart every time.
  struct Walker {
    uint32_t x, y, imageAt, deltaAt, p;
  } at[2];
#pragma unroll
  for (int h = 0; h != 2; ++h) {
    const uint32_t p = p0 + h * 32 + row;
    const uint32_t pr = a.divOutW(p), b = a.divOutH(pr);
    at[h].x = p - pr * d.outW, at[h].y = pr - b * d.outH;
    at[h].imageAt = b * a.actImageBytes;
    at[h].deltaAt = p * a.deltaPixelBytes;
    at[h].p = p;
  }
  const uint32_t tapY = kh - uint32_t(d.padH), tapX = kw - uint32_t(d.padW);
  auto load = [&](char *__restrict__ into) {
    char *stage = into + wave * 1024;
#pragma unroll
    for (int h = 0; h != 2; ++h) {
      Walker &w = at[h];
      const uint32_t iy = w.y * d.strideH + tapY, ix = w.x * d.strideW + tapX;
      const bool inside = w.p < p1;
      const uint32_t deltaAt = inside ? w.deltaAt : kWuInvalid;
      const uint32_t actAt =
          inside && iy - d.loH < d.hiH - d.loH && ix - d.loW < d.hiW - d.loW
              ? w.imageAt + (iy * d.inW + ix) * a.actPixelBytes
              : kWuInvalid;
      // (any sum with a kWuInvalid in it lies beyond the buffer and reads
      // as zeros)
      loadToLds(deltaBuf, (LdsPtr)(stage + (2 * h) * kWuTileBytes),
                deltaAt + deltaLane, 0);
      loadToLds(actBuf, (LdsPtr)(stage + (2 * h + 1) * kWuTileBytes),
                actAt + actLane, 0);
      // 64 pixels on: stepX columns, stepY rows, stepImages images, with the
      // carries (a single one each: x < outW and stepX < outW, likewise y)
      w.p += 64, w.deltaAt += 64 * a.deltaPixelBytes;
      w.x += a.stepX;
      const uint32_t carryX = w.x >= d.outW ? 1u : 0u;
      w.x -= carryX ? d.outW : 0u;
      w.y += a.stepY + carryX;
      const uint32_t carryY = w.y >= d.outH ? 1u : 0u;
      w.y -= carryY ? d.outH : 0u;
      w.imageAt += (a.stepImages + carryY) * a.actImageBytes;
    }
  };

  // Reads.  For a block of 16 channels starting at chunk 2 blk of the tile,
  // lane l = (quarter b = l / 16, i = l % 16) points at row 8 b + i / 4 and
  // the 8 bytes of channels 4 (i % 4) .. + 3.
  const uint32_t rb = lane >> 4, ri = lane & 15;
  const uint32_t readRow = 8 * rb + (ri >> 2);
  const uint32_t readSwizzle = 2 * ((ri >> 2) + 4 * (rb & 1));
  uint32_t deltaOff[4], actOff[4];
#pragma unroll
  for (int blk = 0; blk != 4; ++blk) {
    const uint32_t dChunk = 2 * (wm * 4 + blk) + ((ri & 3) >> 1);
    const uint32_t aChunk = 2 * (wn * 4 + blk) + ((ri & 3) >> 1);
    deltaOff[blk] =
        readRow * 256 + ((dChunk ^ readSwizzle) * 16) + 8 * (ri & 1);
    actOff[blk] = kWuTileBytes + readRow * 256 +
                  ((aChunk ^ readSwizzle) * 16) + 8 * (ri & 1);
  }

  floatx4 acc[4][4];
#pragma unroll
  for (int i = 0; i != 4; ++i)
#pragma unroll
    for (int j = 0; j != 4; ++j)
      acc[i][j] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

  // Software pipeline.  Iteration `step`: wait for step + 1's tiles, issue
  // the loads of step + kWuStages into the stage that step's operands were
  // read from (in the iteration before), read step + 1's operands, and only
  // then multiply step's, so that the reads run under the MFMAs.  (What the
  // loop waits for is the loads: the nine taps of a chunk read the same
  // pixels on nine XCDs, nine in ten L2 requests miss, and an XCD's link to
  // memory delivers about 1.3 TB/s.)
  // (`__restrict__` on the stage written and the stage read, so that the
  // compiler does not make the reads wait for the loads just issued: a load
  // that writes LDS is a pending LDS write to it.)
  struct Operands {
    half8 da[4], ab[4];
  };
  auto read = [&](Operands &o, const char *__restrict__ tile) {
#pragma unroll
    for (int blk = 0; blk != 4; ++blk)
      o.da[blk] = transposedOperand(tile + deltaOff[blk]);
#pragma unroll
    for (int blk = 0; blk != 4; ++blk)
      o.ab[blk] = transposedOperand(tile + actOff[blk]);
  };
  auto multiply = [&](const Operands &o) {
#pragma unroll
    for (int i = 0; i != 4; ++i)
#pragma unroll
      for (int j = 0; j != 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(o.da[i], o.ab[j],
                                                           acc[i][j], 0, 0, 0);
  };
  auto tileOf = [&](uint32_t step) {
    return lds + (step % kWuStages) * kWuStageBytes + grp * 2 * kWuTileBytes;
  };
  // (No branches in the loop: loads are issued for steps beyond the chunk's
  // last too - all out of range, they write zeros - and an odd count of steps
  // is rounded up, the extra one multiplying zeros.  So the loads of exactly
  // two steps, 4 each, are behind the one waited for.)
  auto iteration = [&](uint32_t step, const Operands &cur, Operands &next,
                       char *__restrict__ into,
                       const char *__restrict__ from) {
    MXK_WAIT_VMCNT(8);
    stepBarrier();
    // (everybody's reads of step's stage finished an iteration ago)
    load(into);
    read(next, from);
    multiply(cur);
    MXK_WAIT_LGKMCNT0();
  };
#pragma unroll
  for (int s = 0; s != kWuStages; ++s)
    load(lds + s * kWuStageBytes);
  Operands even, odd;
  MXK_WAIT_VMCNT(12);
  stepBarrier();
  read(even, tileOf(0));
  MXK_WAIT_LGKMCNT0();
  for (uint32_t step = 0; step < steps; step += 2) {
    iteration(step, even, odd, lds + (step % kWuStages) * kWuStageBytes,
              tileOf(step + 1));
    iteration(step + 1, odd, even,
              lds + ((step + 1) % kWuStages) * kWuStageBytes,
              tileOf(step + 2));
  }
  MXK_WAIT_VMCNT(0);

  // The second half's waves hand their sums to the first half's, which add
  // them and lay the tile out as [ci][co] rows; then everybody stores rows.
  __syncthreads();
  uintx4 *exchange = reinterpret_cast<uintx4 *>(lds);
  char *tileOut = lds + 4 * 16 * 1024;
  if (grp == 1) {
#pragma unroll
    for (int i = 0; i != 4; ++i)
#pragma unroll
      for (int j = 0; j != 4; ++j)
        exchange[((wave & 3) * 16 + i * 4 + j) * 64 + lane] =
            __builtin_bit_cast(uintx4, acc[i][j]);
  }
  __syncthreads();
  if (grp == 0) {
    // lane: ci = 16 j + lane % 16 of the wave's 64, co = 16 i + 4 (lane / 16)
    // + v
#pragma unroll
    for (int i = 0; i != 4; ++i)
#pragma unroll
      for (int j = 0; j != 4; ++j) {
        const floatx4 other = __builtin_bit_cast(
            floatx4, exchange[((wave & 3) * 16 + i * 4 + j) * 64 + lane]);
        const floatx4 sum = acc[i][j] + other;
        const uint32_t ci = wn * 64 + j * 16 + (lane & 15);
        const uint32_t co = wm * 64 + i * 16 + 4 * (lane >> 4);
        *reinterpret_cast<floatx4 *>(tileOut + ci * kWuOutRow + co * 4) = sum;
      }
  }
  __syncthreads();
  float *dst = partial + ((((size_t(chunk) * d.groups + g) * a.taps + tap) *
                               a.ciTiles +
                           ciTile) *
                              a.coTiles +
                          coTile) *
                             (128 * 128);
  // 32 lanes x 16 bytes per row, 16 rows per pass; written through the L2
  // (the other kernel reads the tiles from every XCD, and what is left dirty
  // has to be written back before it starts: 25.8 -> 25.0 us for the pass)
  const __amdgpu_buffer_rsrc_t tileBuf = bufferOf(dst, 128 * 128 * 4);
#pragma unroll
  for (int pass = 0; pass != 8; ++pass) {
    const uint32_t r = pass * 16 + (t >> 5), c = (t & 31) * 4;
    __builtin_amdgcn_raw_buffer_store_b128(
        *reinterpret_cast<const uintx4 *>(tileOut + r * kWuOutRow + c * 4),
        tileBuf, (r * 128 + c) * 4, 0, kWriteThroughStore);
  }
}

/// deltas[g][co][ci][tap] = sum over the chunks in a fixed order.  Four
/// neighbouring lanes share an output vector of four channels: lane part p
/// adds the chunks p, p + 4, ... (two running sums, two loads in flight), and
/// the four meet as (s0 + s1) + (s2 + s3) - four times the threads of a lane
/// per output, which is what a 16 MB stream needs to keep HBM busy.
/// (Measured alternatives, all slower: one lane per output vector with four
/// running sums - 6.3 us; two outputs per thread with eight sums; a workgroup
/// per input channel that gathers each output channel's taps in LDS and
/// writes them together.)
template <class OutT>
__global__ __launch_bounds__(256) void wuTapSumKernel(
    const float *__restrict__ partial, OutT *__restrict__ out, uint32_t chunks,
    uint32_t groups, uint32_t taps, uint32_t ci, uint32_t co,
    uint32_t ciTiles, uint32_t coTiles) {
  // thread -> (group, tap, ci, 4 co, part), part fastest
  const uint64_t id = (uint64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> 2;
  const uint32_t part = threadIdx.x & 3;
  const uint32_t co4 = (coTiles * 128) / 4;
  const uint32_t c = uint32_t(id % co4) * 4;
  uint64_t rest = id / co4;
  const uint32_t i = uint32_t(rest % (ciTiles * 128));
  rest /= ciTiles * 128;
  const uint32_t tap = uint32_t(rest % taps);
  const uint32_t g = uint32_t(rest / taps);
  // (whole groups of four lanes leave together)
  if (g >= groups || i >= ci || c >= co)
    return;
  const size_t tile = 128 * 128;
  const size_t perChunk = size_t(groups) * taps * ciTiles * coTiles * tile;
  const float *src = partial +
                     (((size_t(g) * taps + tap) * ciTiles + i / 128) * coTiles +
                      c / 128) *
                         tile +
                     (i % 128) * 128 + c % 128;
  float4 sum[2] = {};
  uint32_t p = part;
  for (; p + 4 < chunks; p += 8) {
    const float4 v0 = *reinterpret_cast<const float4 *>(src + size_t(p) * perChunk);
    const float4 v1 =
        *reinterpret_cast<const float4 *>(src + size_t(p + 4) * perChunk);
    sum[0].x += v0.x, sum[0].y += v0.y, sum[0].z += v0.z, sum[0].w += v0.w;
    sum[1].x += v1.x, sum[1].y += v1.y, sum[1].z += v1.z, sum[1].w += v1.w;
  }
  if (p < chunks) {
    const float4 v0 = *reinterpret_cast<const float4 *>(src + size_t(p) * perChunk);
    sum[0].x += v0.x, sum[0].y += v0.y, sum[0].z += v0.z, sum[0].w += v0.w;
  }
  float v[4] = {sum[0].x + sum[1].x, sum[0].y + sum[1].y, sum[0].z + sum[1].z,
                sum[0].w + sum[1].w};
#pragma unroll
  for (int e = 0; e != 4; ++e) {
    v[e] += __shfl_xor(v[e], 1); // s0 + s1, s2 + s3
    v[e] += __shfl_xor(v[e], 2);
  }
  // (co is a multiple of 8: the planner's condition); lane part p stores
  // channel c + p
  storeOut(out, ((size_t(g) * co + c + part) * ci + i) * taps + tap,
           part == 0 ? v[0] : part == 1 ? v[1] : part == 2 ? v[2] : v[3]);
}

uint64_t tilesOf(const WuTapDesc &d) {
  return uint64_t(d.groups) * d.kH * d.kW * ((d.ci + 127) / 128) *
         ((d.co + 127) / 128);
}

} // namespace

bool wuTapTakes(const WuTapDesc &d) {
  const uint64_t M = uint64_t(d.batch) * d.outH * d.outW;
  if (M == 0 || d.ci % 8 != 0 || d.co % 8 != 0 || d.ci == 0 || d.co == 0 ||
      d.kH == 0 || d.kW == 0 || d.strideH == 0 || d.strideW == 0)
    return false;
  const uint64_t actBytes =
      uint64_t(d.batch) * d.inH * d.inW * d.groups * d.ci * 2;
  const uint64_t deltaBytes = M * d.groups * d.co * 2;
  if (actBytes >= kWuInvalid || deltaBytes >= kWuInvalid || M >= kWuInvalid)
    return false;
  if (d.chunkPixels == 0 || d.chunkPixels % 64 != 0)
    return false;
  const uint64_t chunks = (M + d.chunkPixels - 1) / d.chunkPixels;
  return chunks * tilesOf(d) <= 0x7fffffffull &&
         wuTapWorkspaceBytes(d) <= (1ull << 31);
}

uint32_t wuTapChunkPixels(const WuTapDesc &d, uint32_t computeUnits) {
  // About one workgroup per CU; chunks of whole super-steps of 64 pixels, not
  // so short that start-up and the tile's way out outweigh the products.
  // (Dealing the workgroups of a chunk to one XCD, for its L2 to fetch the
  // chunk's pixels once, shortens the loop by a quarter, but the partial
  // tiles' stores, all at the same moment then, take longer than that gains.)
  const uint64_t M = uint64_t(d.batch) * d.outH * d.outW;
  const uint64_t tiles = std::max<uint64_t>(1, tilesOf(d));
  const uint64_t chunks = std::max<uint64_t>(1, computeUnits / tiles);
  uint64_t pixels = (M + chunks - 1) / chunks;
  pixels = std::max<uint64_t>(256, (pixels + 63) / 64 * 64);
  return uint32_t(std::min<uint64_t>(pixels, 1u << 30));
}

uint64_t wuTapWorkspaceBytes(const WuTapDesc &d) {
  const uint64_t M = uint64_t(d.batch) * d.outH * d.outW;
  if (d.chunkPixels == 0)
    return 0;
  const uint64_t chunks = (M + d.chunkPixels - 1) / d.chunkPixels;
  return chunks * tilesOf(d) * 128 * 128 * 4;
}

hipError_t launchWuTap(const WuTapDesc &d, int outType, const void *acts,
                       const void *deltas, void *workspace, void *out,
                       hipStream_t stream) {
  if (!wuTapTakes(d) || (outType != kHalf && outType != kFloat))
    return hipErrorInvalidValue;
  WuTapArgs a{};
  a.d = d;
  a.M = d.batch * d.outH * d.outW;
  a.taps = d.kH * d.kW;
  a.ciTiles = (d.ci + 127) / 128, a.coTiles = (d.co + 127) / 128;
  a.actPixelBytes = d.groups * d.ci * 2;
  a.deltaPixelBytes = d.groups * d.co * 2;
  a.actImageBytes = d.inH * d.inW * a.actPixelBytes;
  a.actBytes = uint64_t(d.batch) * a.actImageBytes;
  a.stepX = 64 % d.outW;
  a.stepY = 64 / d.outW % d.outH;
  a.stepImages = 64 / d.outW / d.outH;
  a.deltaBytes = uint64_t(a.M) * a.deltaPixelBytes;
  a.divOutW = makeFastDiv(d.outW), a.divOutH = makeFastDiv(d.outH);
  a.divTaps = makeFastDiv(a.taps), a.divCiTiles = makeFastDiv(a.ciTiles);
  a.divCoTiles = makeFastDiv(a.coTiles), a.divKW = makeFastDiv(d.kW);
  const uint32_t chunks = (a.M + d.chunkPixels - 1) / d.chunkPixels;
  a.chunks = chunks;
  a.tilesPerChunk = uint32_t(tilesOf(d));
  a.divTilesPerChunk = makeFastDiv(a.tilesPerChunk);
  const uint32_t blocks = chunks * a.tilesPerChunk;
  constexpr int kLds = kWuStages * kWuStageBytes > 64 * 1024 + 128 * kWuOutRow
                           ? kWuStages * kWuStageBytes
                           : 64 * 1024 + 128 * kWuOutRow;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void *>(&wuTapKernel),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
  if (attr != hipSuccess)
    return attr;
  hipLaunchKernelGGL(wuTapKernel, dim3(blocks), dim3(kWuThreads), kLds, stream,
                     a, static_cast<const char *>(acts),
                     static_cast<const char *>(deltas),
                     static_cast<float *>(workspace));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return e;
  const uint64_t threads =
      uint64_t(d.groups) * a.taps * a.ciTiles * 128 * (a.coTiles * 128 / 4) * 4;
  const uint32_t sumBlocks = uint32_t((threads + 255) / 256);
  if (outType == kHalf)
    hipLaunchKernelGGL(wuTapSumKernel<__half>, dim3(sumBlocks), dim3(256), 0,
                       stream, static_cast<const float *>(workspace),
                       static_cast<__half *>(out), chunks, d.groups, a.taps,
                       d.ci, d.co, a.ciTiles, a.coTiles);
  else
    hipLaunchKernelGGL(wuTapSumKernel<float>, dim3(sumBlocks), dim3(256), 0,
                       stream, static_cast<const float *>(workspace),
                       static_cast<float *>(out), chunks, d.groups, a.taps,
                       d.ci, d.co, a.ciTiles, a.coTiles);
  return hipGetLastError();
}

} // namespace mxk

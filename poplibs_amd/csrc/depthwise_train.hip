// Depthwise kernels for the training passes of a depthwise layer (one input
// and one output channel per group, channels-last, fp16 data, fp32 sums):
//
//   depthwiseDirectKernel      a forward convolution that also takes a
//                              dilated (zero-stuffed) input, which is what
//                              the backward pass of a strided depthwise layer
//                              is; one thread per output pixel and vector of
//                              8 channels, taps that fall between input
//                              elements skipped.
//   depthwiseWeightDeltaKernel the gradient with respect to the weights,
//                              dW[tap][c] = sum over batch and output pixels
//                              of deltas[pixel][c] * acts[pixel under tap][c];
//                              one thread per (tap, vector of 8 channels),
//                              walking a slice of the pixels; the per-slice
//                              sums go to a workspace and a second kernel
//                              adds the slices in order.
//
// Both are bound by memory: they read each operand from HBM once (re-reads
// of neighbouring taps hit the caches) and have no matrix-core work.  They
// take the role of PopLibs' HorizontalMac vertices in the backward and weight
// update passes (lib/poplin/codelets/ConvPartialHorizontalMac.cpp:34-133).
#include "device_types.hpp"
#include "kernels.hpp"

#include <algorithm>

namespace mxk {
namespace {

union Vec8 {
  uint4 raw;
  __half2 h2[4];
};

__device__ __forceinline__ void fma8(float (&acc)[8], const Vec8 &x,
                                     const Vec8 &k) {
#pragma unroll
  for (int i = 0; i != 4; ++i) {
    const float2 xf = __half22float2(x.h2[i]);
    const float2 kf = __half22float2(k.h2[i]);
    acc[2 * i] = fmaf(xf.x, kf.x, acc[2 * i]);
    acc[2 * i + 1] = fmaf(xf.y, kf.y, acc[2 * i + 1]);
  }
}

__device__ __forceinline__ void store8(__half *p, const float (&v)[8]) {
  Vec8 o;
#pragma unroll
  for (int i = 0; i != 4; ++i)
    o.h2[i] = roundPairToHalf(v[2 * i], v[2 * i + 1]);
  *reinterpret_cast<uint4 *>(p) = o.raw;
}
__device__ __forceinline__ void store8(float *p, const float (&v)[8]) {
  *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<float4 *>(p + 4) = float4{v[4], v[5], v[6], v[7]};
}

// The same for fp32 inputs: a 16-byte vector holds four channels.
__device__ __forceinline__ void fma4(float (&acc)[4], const uint4 &x,
                                     const uint4 &k) {
  acc[0] = fmaf(__uint_as_float(x.x), __uint_as_float(k.x), acc[0]);
  acc[1] = fmaf(__uint_as_float(x.y), __uint_as_float(k.y), acc[1]);
  acc[2] = fmaf(__uint_as_float(x.z), __uint_as_float(k.z), acc[2]);
  acc[3] = fmaf(__uint_as_float(x.w), __uint_as_float(k.w), acc[3]);
}
__device__ __forceinline__ void store4(float *p, const float (&v)[4]) {
  *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void store4(__half *p, const float (&v)[4]) {
  const __half2 lo = roundPairToHalf(v[0], v[1]),
                hi = roundPairToHalf(v[2], v[3]);
  *reinterpret_cast<uint2 *>(p) = uint2{__builtin_bit_cast(uint32_t, lo),
                                        __builtin_bit_cast(uint32_t, hi)};
}

struct DirectArgs {
  DepthwiseDesc d;
  FastDiv divVecs, divOutW, divOutH, divInDilH, divInDilW;
  uint32_t vecs;
  uint64_t items; // batch * outH * outW * vecs
};

/// InT: __half (vectors of 8 channels) or float (of 4).
template <class OutT, class InT = __half>
__global__ __launch_bounds__(256) void depthwiseDirectKernel(
    DirectArgs a, const InT *__restrict__ in, const InT *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out) {
  constexpr int E = 16 / int(sizeof(InT));
  const DepthwiseDesc &d = a.d;
  const uint64_t item = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (item >= a.items)
    return;
  // item = ((b * outH + oh) * outW + ow) * vecs + v
  const uint32_t pixel = a.divVecs(uint32_t(item));
  const uint32_t v = uint32_t(item) - pixel * a.vecs;
  const uint32_t row = a.divOutW(pixel);
  const uint32_t ow = pixel - row * d.outW;
  const uint32_t b = a.divOutH(row);
  const uint32_t oh = row - b * d.outH;
  const uint32_t c = v * E;
  float acc[E];
#pragma unroll
  for (int i = 0; i != E; ++i)
    acc[i] = bias ? Load<OutT>::at(bias, c + i, 0) : 0.0f;
  const int ihBase = int(oh * d.strideH) - d.padH;
  const int iwBase = int(ow * d.strideW) - d.padW;
  const InT *image = in + size_t(b) * d.inH * d.inW * d.channels + c;
  // Validity is separable: the kernel columns that read an input element
  // are worked out once (a bit each - up to 32 columns at a time), then for
  // every valid kernel row only those columns are visited.
  for (uint32_t kw0 = 0; kw0 < d.kW; kw0 += 32) {
    uint32_t columns = 0;
    const uint32_t kwEnd = min(d.kW - kw0, 32u);
    for (uint32_t j = 0; j != kwEnd; ++j) {
      const int iwD = iwBase + int((kw0 + j) * d.dilW);
      const uint32_t iw = a.divInDilW(uint32_t(iwD));
      if (iwD >= 0 && iw * d.inDilW == uint32_t(iwD) && iw >= d.loW &&
          iw < d.hiW)
        columns |= 1u << j;
    }
    if (columns == 0)
      continue;
    for (uint32_t kh = 0; kh != d.kH; ++kh) {
      const int ihD = ihBase + int(kh * d.dilH);
      const uint32_t ih = a.divInDilH(uint32_t(ihD));
      if (ihD < 0 || ih * d.inDilH != uint32_t(ihD) || ih < d.loH ||
          ih >= d.hiH)
        continue;
      const InT *row = image + size_t(ih) * d.inW * d.channels;
      const InT *taps = w + size_t(kh * d.kW + kw0) * d.channels + c;
      for (uint32_t rest = columns; rest != 0; rest &= rest - 1) {
        const uint32_t j = uint32_t(__ffs(int(rest))) - 1;
        const uint32_t iw =
            a.divInDilW(uint32_t(iwBase + int((kw0 + j) * d.dilW)));
        Vec8 x, k;
        x.raw = *reinterpret_cast<const uint4 *>(row + size_t(iw) * d.channels);
        k.raw = *reinterpret_cast<const uint4 *>(taps + size_t(j) * d.channels);
        if constexpr (E == 8)
          fma8(acc, x, k);
        else
          fma4(acc, x.raw, k.raw);
      }
    }
  }
  if constexpr (E == 8)
    store8(out + size_t(pixel) * d.channels + c, acc);
  else
    store4(out + size_t(pixel) * d.channels + c, acc);
}

struct BlockArgs {
  DepthwiseDesc d;
  FastDiv divVecs, divBlocksW, divStrips;
  uint32_t vecs, blocksW, strips;
  int32_t firstBlockH, firstBlockW;
  uint64_t items; // batch * strips * blocksW * vecs
};

/// The same convolution for an input dilated by S in both dimensions with
/// unit stride and unit kernel dilation (the backward pass of a layer of
/// stride S), K x K taps.  With oh - padH = S q + r (0 <= r < S) the taps
/// that read an input element are those with (r + kh) % S == 0, and they read
/// row q + (r + kh) / S: the same for every output of phase r.  So a thread
/// takes S x S blocks of outputs (one output of every phase), R blocks below
/// each other, for one vector of 8 channels: it loads the (R + ND - 1) x ND
/// input vectors they need (ND = (K + S - 2) / S + 1) and all K x K taps
/// once, and every output then takes exactly its own taps - no tests, no
/// divergence between neighbouring outputs, each input vector loaded once per
/// thread.
template <int S, int K, int R, class OutT>
__global__ __launch_bounds__(256) void depthwiseDilatedBlockKernel(
    BlockArgs a, const __half *__restrict__ in, const __half *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out) {
  const DepthwiseDesc &d = a.d;
  const uint64_t item = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (item >= a.items)
    return;
  // item = ((b * strips + strip) * blocksW + block column) * vecs + v
  const uint32_t col = a.divVecs(uint32_t(item));
  const uint32_t v = uint32_t(item) - col * a.vecs;
  const uint32_t t = a.divBlocksW(col);
  const uint32_t bw = col - t * a.blocksW;
  const uint32_t b = a.divStrips(t);
  const uint32_t strip = t - b * a.strips;
  const int qw = a.firstBlockW + int(bw);
  const int qh0 = a.firstBlockH + int(strip) * R;
  const uint32_t c = v * 8;
  constexpr int ND = (K + S - 2) / S + 1;
  constexpr int ROWS = R + ND - 1;

  const __half *image = in + size_t(b) * d.inH * d.inW * d.channels + c;
  Vec8 x[ROWS][ND];
#pragma unroll
  for (int i = 0; i != ROWS; ++i)
#pragma unroll
    for (int j = 0; j != ND; ++j) {
      const int ih = qh0 + i, iw = qw + j;
      x[i][j].raw = uint4{0, 0, 0, 0};
      if (ih >= int(d.loH) && ih < int(d.hiH) && iw >= int(d.loW) &&
          iw < int(d.hiW))
        x[i][j].raw = *reinterpret_cast<const uint4 *>(
            image + (size_t(ih) * d.inW + size_t(iw)) * d.channels);
    }
  Vec8 k[K * K];
#pragma unroll
  for (int tap = 0; tap != K * K; ++tap)
    k[tap].raw =
        *reinterpret_cast<const uint4 *>(w + size_t(tap) * d.channels + c);
  float biasV[8];
#pragma unroll
  for (int i = 0; i != 8; ++i)
    biasV[i] = bias ? Load<OutT>::at(bias, c + i, 0) : 0.0f;

  OutT *outImage = out + size_t(b) * d.outH * d.outW * d.channels + c;
#pragma unroll
  for (int i = 0; i != R; ++i)
#pragma unroll
    for (int rh = 0; rh != S; ++rh) {
      const int oh = S * (qh0 + i) + rh + d.padH;
      if (oh < 0 || oh >= int(d.outH))
        continue;
#pragma unroll
      for (int rw = 0; rw != S; ++rw) {
        const int ow = S * qw + rw + d.padW;
        if (ow < 0 || ow >= int(d.outW))
          continue;
        float acc[8];
#pragma unroll
        for (int e = 0; e != 8; ++e)
          acc[e] = biasV[e];
#pragma unroll
        for (int kh = 0; kh != K; ++kh)
#pragma unroll
          for (int kw = 0; kw != K; ++kw)
            if ((rh + kh) % S == 0 && (rw + kw) % S == 0)
              fma8(acc, x[i + (rh + kh) / S][(rw + kw) / S], k[kh * K + kw]);
        store8(outImage + (size_t(oh) * d.outW + size_t(ow)) * d.channels,
               acc);
      }
    }
}

inline int floorDiv(int n, int d) { return n >= 0 ? n / d : -((-n + d - 1) / d); }

/// Launches depthwiseDilatedBlockKernel<S, K, R> on a shape it is built for.
template <int S, int K, int R>
hipError_t launchDilatedBlock(const DepthwiseDesc &d, int outType,
                              const void *in, const void *w, const void *bias,
                              void *out, hipStream_t stream) {
  BlockArgs a;
  a.d = d;
  a.vecs = d.channels / 8;
  a.firstBlockH = floorDiv(-d.padH, S);
  a.firstBlockW = floorDiv(-d.padW, S);
  const uint32_t blocksH =
      uint32_t(floorDiv(int(d.outH) - 1 - d.padH, S) - a.firstBlockH + 1);
  a.blocksW =
      uint32_t(floorDiv(int(d.outW) - 1 - d.padW, S) - a.firstBlockW + 1);
  a.strips = (blocksH + R - 1) / R;
  a.items = uint64_t(d.batch) * a.strips * a.blocksW * a.vecs;
  if (a.items >= (1ull << 31))
    return hipErrorInvalidConfiguration;
  a.divVecs = makeFastDiv(a.vecs);
  a.divBlocksW = makeFastDiv(a.blocksW);
  a.divStrips = makeFastDiv(a.strips);
  const dim3 grid{uint32_t((a.items + 255) / 256)}, block{256};
  if (outType == kHalf)
    hipLaunchKernelGGL((depthwiseDilatedBlockKernel<S, K, R, __half>), grid,
                       block, 0, stream, a, static_cast<const __half *>(in),
                       static_cast<const __half *>(w),
                       static_cast<const __half *>(bias),
                       static_cast<__half *>(out));
  else
    hipLaunchKernelGGL((depthwiseDilatedBlockKernel<S, K, R, float>), grid,
                       block, 0, stream, a, static_cast<const __half *>(in),
                       static_cast<const __half *>(w),
                       static_cast<const float *>(bias),
                       static_cast<float *>(out));
  return hipGetLastError();
}

struct DeltaArgs {
  DepthwiseDesc d;     // the FORWARD convolution
  FastDiv divVecs, divOutW, divOutH;
  uint32_t vecs, taps;
  uint32_t items;      // taps * vecs
  uint32_t itemsPerBlock, slots; // itemsPerBlock * slots <= 256 threads
  uint32_t pixels;     // batch * outH * outW
  uint32_t pixelsPerSlice, pixelsPerSlot, slices;
};

/// partial[slice][tap][c] = sum over the slice's output pixels.  A workgroup
/// takes itemsPerBlock (tap, channel vector) items and one slice of the
/// pixels; when there are few items, `slots` groups of threads walk a part of
/// the slice each and their sums meet in LDS.
/// InT: __half (vectors of 8 channels) or float (of 4).
template <class InT>
__global__ __launch_bounds__(256) void depthwiseWeightDeltaKernel(
    DeltaArgs a, const InT *__restrict__ acts, const InT *__restrict__ deltas,
    float *__restrict__ partial) {
  constexpr int E = 16 / int(sizeof(InT));
  __shared__ float meet[256][9]; // 8 sums per thread, padded
  const DepthwiseDesc &d = a.d;
  const uint32_t slot = threadIdx.x / a.itemsPerBlock;
  const uint32_t itemLocal = threadIdx.x - slot * a.itemsPerBlock;
  const uint32_t item = blockIdx.x * a.itemsPerBlock + itemLocal;
  const bool active = slot < a.slots && item < a.items;
  // item = tap * vecs + v: neighbouring threads read neighbouring channels
  const uint32_t tap = a.divVecs(active ? item : 0);
  const uint32_t c = ((active ? item : 0) - tap * a.vecs) * E;
  const uint32_t kh = tap / d.kW, kw = tap - kh * d.kW;
  const uint32_t slice = blockIdx.y;
  const uint32_t sliceEnd =
      min((slice + 1) * a.pixelsPerSlice, a.pixels);
  const uint32_t first =
      min(slice * a.pixelsPerSlice + slot * a.pixelsPerSlot, sliceEnd);
  const uint32_t last = active ? min(first + a.pixelsPerSlot, sliceEnd) : first;
  // (b, oh, ow) of the first pixel; they advance without dividing
  uint32_t row = a.divOutW(first);
  uint32_t ow = first - row * d.outW;
  uint32_t b = a.divOutH(row);
  uint32_t oh = row - b * d.outH;
  const int khd = int(kh * d.dilH) - d.padH, kwd = int(kw * d.dilW) - d.padW;
  float acc[E] = {};
  // Four pixels a round: their loads are issued together, so that a wave has
  // eight of them in flight (the walk is bound by load latency, not by
  // arithmetic).
  constexpr int kUnroll = 4;
  for (uint32_t p = first; p < last; p += kUnroll) {
    Vec8 x[kUnroll], z[kUnroll];
#pragma unroll
    for (int u = 0; u != kUnroll; ++u) {
      const int ih = int(oh * d.strideH) + khd, iw = int(ow * d.strideW) + kwd;
      const bool ok = p + u < last && ih >= int(d.loH) && ih < int(d.hiH) &&
                      iw >= int(d.loW) && iw < int(d.hiW);
      x[u].raw = uint4{0, 0, 0, 0};
      z[u].raw = uint4{0, 0, 0, 0};
      if (ok) {
        x[u].raw = *reinterpret_cast<const uint4 *>(
            acts +
            ((size_t(b) * d.inH + uint32_t(ih)) * d.inW + uint32_t(iw)) *
                d.channels +
            c);
        z[u].raw = *reinterpret_cast<const uint4 *>(
            deltas + size_t(p + u) * d.channels + c);
      }
      if (++ow == d.outW) {
        ow = 0;
        if (++oh == d.outH) {
          oh = 0;
          ++b;
        }
      }
    }
#pragma unroll
    for (int u = 0; u != kUnroll; ++u) {
      if constexpr (E == 8)
        fma8(acc, x[u], z[u]);
      else
        fma4(acc, x[u].raw, z[u].raw);
    }
  }
  if (a.slots > 1) {
#pragma unroll
    for (int i = 0; i != E; ++i)
      meet[threadIdx.x][i] = acc[i];
    __syncthreads();
    if (slot == 0)
      for (uint32_t s2 = 1; s2 != a.slots; ++s2)
#pragma unroll
        for (int i = 0; i != E; ++i)
          acc[i] += meet[s2 * a.itemsPerBlock + itemLocal][i];
  }
  if (!active || slot != 0)
    return;
  float *dst = partial + (size_t(slice) * a.taps + tap) * d.channels + c;
#pragma unroll
  for (int i = 0; i != E; i += 4)
    *reinterpret_cast<float4 *>(dst + i) =
        float4{acc[i], acc[i + 1], acc[i + 2], acc[i + 3]};
}

/// out[c][tap] = sum over slices of partial[slice][tap][c], in a fixed order:
/// a workgroup of 16 waves takes 16 outputs and cuts the slices into 64
/// contiguous parts, a quarter of a wave (16 lanes, 64 contiguous bytes per
/// slice) to each; a lane adds up its part with sixteen loads in flight, then
/// one thread per output adds the 64 sums in order.  Few outputs per
/// workgroup, because the outputs are few (taps x channels) and the walk over
/// the slices is a chain of memory latencies: this way there are four times
/// the workgroups and a quarter of the chain.
template <class OutT>
__global__ __launch_bounds__(1024) void depthwiseDeltaSumKernel(
    const float *__restrict__ partial, uint32_t slices, uint32_t taps,
    uint32_t channels, OutT *__restrict__ out) {
  __shared__ float meet[64][16];
  const uint32_t column = threadIdx.x % 16, part = threadIdx.x / 16;
  const uint32_t outputs = taps * channels;
  const uint32_t i = blockIdx.x * 16 + column; // tap * C + c
  const uint32_t per = (slices + 63) / 64;
  const uint32_t from = min(part * per, slices), to = min(from + per, slices);
  constexpr int kInFlight = 16;
  float sum[kInFlight] = {};
  if (i < outputs) {
    uint32_t s = from;
    for (; s + kInFlight <= to; s += kInFlight)
#pragma unroll
      for (int u = 0; u != kInFlight; ++u)
        sum[u] += partial[size_t(s + u) * outputs + i];
#pragma unroll
    for (int u = 0; u != kInFlight - 1; ++u)
      if (s + u < to)
        sum[u] += partial[size_t(s + u) * outputs + i];
  }
#pragma unroll
  for (int width = kInFlight / 2; width != 0; width /= 2)
#pragma unroll
    for (int u = 0; u != width; ++u)
      sum[u] += sum[u + width];
  // The 64 sums of an output meet in two steps of eight, each in order (one
  // thread adding all 64 is a chain of 64 LDS reads at the kernel's end).
  meet[part][column] = sum[0];
  __syncthreads();
  float eight = 0.0f;
  if (part < 8) {
    eight = meet[part * 8][column];
#pragma unroll
    for (int w = 1; w != 8; ++w)
      eight += meet[part * 8 + w][column];
  }
  __syncthreads();
  if (part < 8)
    meet[part][column] = eight;
  __syncthreads();
  if (part != 0 || i >= outputs)
    return;
  float total = meet[0][column];
#pragma unroll
  for (int w = 1; w != 8; ++w)
    total += meet[w][column];
  const uint32_t tap = i / channels, c = i - tap * channels;
  storeOut(out, size_t(c) * taps + tap, total);
}

/// Threads of a workgroup: itemsPerBlock items by `slots` parts of a slice.
void deltaBlockShape(const DepthwiseDesc &d, uint32_t &itemsPerBlock,
                     uint32_t &slots) {
  const uint64_t items =
      uint64_t(d.kH) * d.kW * (uint64_t(d.channels) * d.elemBytes / 16);
  itemsPerBlock = uint32_t(std::min<uint64_t>(std::max<uint64_t>(items, 1), 256));
  slots = 256 / itemsPerBlock;
}

uint32_t deltaSlices(const DepthwiseDesc &d) {
  // About 4 workgroups per CU in all; a slot walks at least 16 pixels.
  uint32_t itemsPerBlock, slots;
  deltaBlockShape(d, itemsPerBlock, slots);
  const uint64_t pixels = uint64_t(d.batch) * d.outH * d.outW;
  const uint64_t items =
      uint64_t(d.kH) * d.kW * (uint64_t(d.channels) * d.elemBytes / 16);
  const uint64_t itemBlocks = (items + itemsPerBlock - 1) / itemsPerBlock;
  uint64_t slices = (1024 + itemBlocks - 1) / std::max<uint64_t>(itemBlocks, 1);
  slices = std::min<uint64_t>(slices, (pixels + 16 * slots - 1) / (16 * slots));
  slices = std::min<uint64_t>(std::max<uint64_t>(slices, 1), 65535);
  return uint32_t(slices);
}

} // namespace

bool depthwiseDirectInBlocks(const DepthwiseDesc &d) {
  return d.inDilH == 2 && d.inDilW == 2 && d.strideH == 1 && d.strideW == 1 &&
         d.dilH == 1 && d.dilW == 1 && d.kH == d.kW &&
         (d.kH == 3 || d.kH == 5) && d.outH < (1u << 30) &&
         d.outW < (1u << 30);
}

hipError_t launchDepthwiseDirect(const DepthwiseDesc &d, int inType,
                                 int outType, const void *in,
                                 const void *weightsPacked, const void *bias,
                                 void *out, hipStream_t stream) {
  const uint32_t perVec = inType == kFloat ? 4 : 8;
  if ((inType != kHalf && inType != kFloat) ||
      d.elemBytes != (inType == kFloat ? 4u : 2u) ||
      d.channels % perVec != 0 || d.inDilH == 0 || d.inDilW == 0)
    return hipErrorInvalidValue;
  DirectArgs a;
  a.d = d;
  a.vecs = d.channels / perVec;
  a.items = uint64_t(d.batch) * d.outH * d.outW * a.vecs;
  if (a.items == 0)
    return hipSuccess;
  // item numbers are divided with 31-bit arithmetic
  if (a.items >= (1ull << 31))
    return hipErrorInvalidConfiguration;
  if (inType == kHalf && (outType == kHalf || outType == kFloat) &&
      depthwiseDirectInBlocks(d)) {
    if (d.kH == 3)
      return launchDilatedBlock<2, 3, 4>(d, outType, in, weightsPacked, bias,
                                         out, stream);
    if (d.kH == 5)
      return launchDilatedBlock<2, 5, 2>(d, outType, in, weightsPacked, bias,
                                         out, stream);
  }
  a.divVecs = makeFastDiv(a.vecs);
  a.divOutW = makeFastDiv(d.outW);
  a.divOutH = makeFastDiv(d.outH);
  a.divInDilH = makeFastDiv(d.inDilH);
  a.divInDilW = makeFastDiv(d.inDilW);
  const dim3 grid{uint32_t((a.items + 255) / 256)}, block{256};
  if (inType == kFloat && outType == kFloat)
    hipLaunchKernelGGL((depthwiseDirectKernel<float, float>), grid, block, 0,
                       stream, a, static_cast<const float *>(in),
                       static_cast<const float *>(weightsPacked),
                       static_cast<const float *>(bias),
                       static_cast<float *>(out));
  else if (inType == kFloat && outType == kHalf)
    hipLaunchKernelGGL((depthwiseDirectKernel<__half, float>), grid, block, 0,
                       stream, a, static_cast<const float *>(in),
                       static_cast<const float *>(weightsPacked),
                       static_cast<const __half *>(bias),
                       static_cast<__half *>(out));
  else if (outType == kHalf)
    hipLaunchKernelGGL(depthwiseDirectKernel<__half>, grid, block, 0, stream, a,
                       static_cast<const __half *>(in),
                       static_cast<const __half *>(weightsPacked),
                       static_cast<const __half *>(bias),
                       static_cast<__half *>(out));
  else if (outType == kFloat)
    hipLaunchKernelGGL(depthwiseDirectKernel<float>, grid, block, 0, stream, a,
                       static_cast<const __half *>(in),
                       static_cast<const __half *>(weightsPacked),
                       static_cast<const float *>(bias),
                       static_cast<float *>(out));
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

size_t depthwiseWeightDeltaWorkspaceBytes(const DepthwiseDesc &d) {
  if (d.dense3x3 == 2)
    return depthwiseRowsDeltaWorkspaceBytes(d);
  return size_t(deltaSlices(d)) * d.kH * d.kW * d.channels * sizeof(float);
}

hipError_t launchDepthwiseWeightDeltas(const DepthwiseDesc &d, int outType,
                                       const void *acts, const void *deltas,
                                       void *workspace, void *weightDeltas,
                                       hipStream_t stream) {
  // half tensors, or fp32 ones (the slices' walk only)
  const uint32_t perVec = 16 / d.elemBytes;
  if ((d.elemBytes != 2 && d.elemBytes != 4) || d.channels % perVec != 0 ||
      d.inDilH != 1 || d.inDilW != 1 || (d.elemBytes == 4 && d.dense3x3 == 2))
    return hipErrorInvalidValue;
  DeltaArgs a;
  a.d = d;
  a.vecs = d.channels / perVec;
  a.taps = d.kH * d.kW;
  const uint64_t items = uint64_t(a.taps) * a.vecs;
  const uint64_t pixels = uint64_t(d.batch) * d.outH * d.outW;
  if (items == 0)
    return hipSuccess;
  if (items >= (1ull << 31) || pixels >= (1ull << 31) || !workspace)
    return hipErrorInvalidConfiguration;
  a.items = uint32_t(items);
  a.pixels = uint32_t(pixels);
  float *partial = static_cast<float *>(workspace);
  if (d.dense3x3 == 2) {
    // persistent workgroups with the rows in LDS rings: one tile each
    const hipError_t e = launchDepthwiseRowsDeltas(d, acts, deltas, partial,
                                                   &a.slices, stream);
    if (e != hipSuccess)
      return e;
  } else {
    a.slices = deltaSlices(d);
    deltaBlockShape(d, a.itemsPerBlock, a.slots);
    a.pixelsPerSlice = uint32_t((pixels + a.slices - 1) / a.slices);
    a.pixelsPerSlot = (a.pixelsPerSlice + a.slots - 1) / a.slots;
    a.divVecs = makeFastDiv(a.vecs);
    a.divOutW = makeFastDiv(d.outW);
    a.divOutH = makeFastDiv(d.outH);
    const dim3 grid{uint32_t((items + a.itemsPerBlock - 1) / a.itemsPerBlock),
                    a.slices},
        block{256};
    if (d.elemBytes == 4)
      hipLaunchKernelGGL(depthwiseWeightDeltaKernel<float>, grid, block, 0,
                         stream, a, static_cast<const float *>(acts),
                         static_cast<const float *>(deltas), partial);
    else
      hipLaunchKernelGGL(depthwiseWeightDeltaKernel<__half>, grid, block, 0,
                         stream, a, static_cast<const __half *>(acts),
                         static_cast<const __half *>(deltas), partial);
  }
  const uint32_t outputs = a.taps * d.channels;
  const dim3 grid2{(outputs + 15) / 16};
  const dim3 block2{1024};
  if (outType == kHalf)
    hipLaunchKernelGGL(depthwiseDeltaSumKernel<__half>, grid2, block2, 0, stream,
                       partial, a.slices, a.taps, d.channels,
                       static_cast<__half *>(weightDeltas));
  else if (outType == kFloat)
    hipLaunchKernelGGL(depthwiseDeltaSumKernel<float>, grid2, block2, 0, stream,
                       partial, a.slices, a.taps, d.channels,
                       static_cast<float *>(weightDeltas));
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

} // namespace mxk

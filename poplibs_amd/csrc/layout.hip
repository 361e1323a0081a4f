// Layout conversions between the external tensor layouts of the convolution
// API ([B][G*C][field...] activations, [G][Co][Ci][kernel...] weights) and the
// device layouts the kernels use, plus the stand-alone bias add.  None of
// these sit on the timed path: tensors live in the device layout.
#include "device_types.hpp"
#include "kernels.hpp"

namespace mxk {
namespace {

struct PermuteArgs {
  uint64_t dstDims[4];
  uint64_t srcStride[4]; // stride in the source of each destination dimension
  uint64_t total;
};

template <class T>
__global__ __launch_bounds__(256) void permuteKernel(PermuteArgs a,
                                                     const T *__restrict__ src,
                                                     T *__restrict__ dst) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= a.total)
    return;
  uint64_t rest = tid, srcIndex = 0;
  for (int j = 3; j >= 0; --j) {
    srcIndex += (rest % a.dstDims[j]) * a.srcStride[j];
    rest /= a.dstDims[j];
  }
  dst[tid] = src[srcIndex];
}

template <class T>
__global__ __launch_bounds__(256) void packIgemmWeightsKernel(
    const T *__restrict__ src, T *__restrict__ dst, uint32_t co, uint32_t ci,
    uint32_t ciPadded, uint32_t taps, uint32_t coPadded, uint32_t kPadded,
    uint64_t total, bool chansTransposed, bool selected,
    IgemmTapSelection select) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  const uint32_t k = uint32_t(tid % kPadded);
  const uint32_t n = uint32_t((tid / kPadded) % coPadded);
  const uint64_t g = tid / (uint64_t(kPadded) * coPadded);
  T v = T(0);
  const uint32_t packedTaps =
      selected ? select.countD * select.countH * select.countW : taps;
  if (n < co && k < packedTaps * ciPadded) {
    uint32_t tap = k / ciPadded;
    const uint32_t c = k % ciPadded;
    if (selected) {
      const uint32_t j = tap % select.countW, rest = tap / select.countW;
      const uint32_t i = rest % select.countH, plane = rest / select.countH;
      tap = ((select.firstD + plane * select.stepD) * select.kH +
             select.firstH + i * select.stepH) *
                select.kW +
            select.firstW + j * select.stepW;
    }
    // source [G][Co][Ci][taps], or [G][Ci][Co][taps] (a matrix
    // multiplication's right-hand side)
    if (c < ci)
      v = chansTransposed ? src[((g * ci + c) * co + n) * taps + tap]
                          : src[((g * co + n) * ci + c) * taps + tap];
  }
  dst[tid] = v;
}

/// One 16-byte vector of the padded tensor per thread.
template <class T>
__global__ __launch_bounds__(256) void padChansKernel(
    const T *__restrict__ src, T *__restrict__ dst, uint64_t vectors,
    uint32_t ci, uint32_t ciPadded) {
  constexpr uint32_t kVec = 16 / sizeof(T);
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= vectors)
    return;
  const uint32_t perGroup = ciPadded / kVec;
  const uint64_t pg = tid / perGroup; // pixel * groups + group
  const uint32_t c0 = uint32_t(tid - pg * perGroup) * kVec;
  union {
    T e[kVec];
    uint4 u;
  } v;
#pragma unroll
  for (uint32_t i = 0; i != kVec; ++i)
    v.e[i] = c0 + i < ci ? src[pg * ci + c0 + i] : T(0);
  reinterpret_cast<uint4 *>(dst)[tid] = v.u;
}

struct FlipArgs {
  uint64_t co, ci, taps, total;
  uint32_t numDims;
  uint32_t shape[kMaxDims];
};

template <class T>
__global__ __launch_bounds__(256) void transposeChansFlipKernel(
    FlipArgs a, const T *__restrict__ src, T *__restrict__ dst) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= a.total)
    return;
  // tid indexes dst [g][ci][co][k]
  uint64_t r = tid;
  const uint64_t k = r % a.taps;
  r /= a.taps;
  const uint64_t co = r % a.co;
  r /= a.co;
  const uint64_t ci = r % a.ci;
  const uint64_t g = r / a.ci;
  // reverse every axis of the row-major tap index
  uint64_t rem = k, flipped = 0, stride = 1;
  for (int d = int(a.numDims) - 1; d >= 0; --d) {
    const uint64_t x = rem % a.shape[d];
    rem /= a.shape[d];
    flipped += (a.shape[d] - 1 - x) * stride;
    stride *= a.shape[d];
  }
  dst[tid] = src[((g * a.co + co) * a.ci + ci) * a.taps + flipped];
}

template <class T>
__global__ __launch_bounds__(256) void addBiasKernel(T *acts,
                                                     const T *__restrict__ bias,
                                                     uint64_t total,
                                                     uint64_t channels) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  const float v = Load<T>::at(acts, tid, 0) + Load<T>::at(bias, tid % channels, 0);
  storeOut(acts, tid, v);
}

template <typename T>
__global__ __launch_bounds__(256) void scaledAddKernel(T *a,
                                                       float scaleA,
                                                       const T *__restrict__ b,
                                                       float scaleB,
                                                       uint64_t total) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  storeOut(a, tid,
           scaleA * Load<T>::at(a, tid, 0) + scaleB * Load<T>::at(b, tid, 0));
}

constexpr uint32_t kSwapChans = 64, kSwapRows = 128;

struct SwapArgs {
  uint32_t batch, pixels, groups, chans; // source [batch][pixels][groups][chans]
  uint32_t pixelsPerTile, batchPerTile;  // their product is kSwapRows
  uint64_t strideG, strideC, strideP;    // destination strides; batch has 1
  uint32_t vectorStores; // 1: 16-byte stores of consecutive batch entries
};

/// dst[g * strideG + c * strideC + p * strideP + b] = src[b][p][g][c]: the
/// batch axis becomes the innermost one.  A workgroup moves a tile of 128
/// (pixel, batch) rows by 64 channels through LDS: loads run along the
/// channels, stores along the batch (and on along the pixels where the
/// destination keeps them adjacent).
template <class T, bool VEC>
__device__ __forceinline__ void
swapBatchChansTile(const SwapArgs &a, const T *__restrict__ src,
                   T *__restrict__ dst, uint32_t blockX, uint32_t blockY,
                   uint32_t blockZ) {
  __shared__ uint32_t tile[kSwapRows][kSwapChans + 1];
  const uint32_t cBlocks = (a.chans + kSwapChans - 1) / kSwapChans;
  const uint32_t c0 = (blockX % cBlocks) * kSwapChans;
  const uint32_t g = blockX / cBlocks;
  const uint32_t p0 = blockY * a.pixelsPerTile;
  const uint32_t b0 = blockZ * a.batchPerTile;
  const uint32_t lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  // row = pLocal * batchPerTile + bLocal
  auto source = [&](uint32_t row, uint32_t c) {
    const uint32_t p = p0 + row / a.batchPerTile;
    const uint32_t b = b0 + row % a.batchPerTile;
    return p < a.pixels && b < a.batch && c < a.chans
               ? src + ((uint64_t(b) * a.pixels + p) * a.groups + g) * a.chans +
                     c
               : nullptr;
  };
  if constexpr (VEC) {
    // 16-byte loads: kVec channels per thread, all loads of a thread issued
    // before the first is used.  The channel count is a multiple of kVec.
    constexpr uint32_t kVec = 16 / sizeof(T);
    constexpr uint32_t kLanesPerRow = kSwapChans / kVec;
    constexpr uint32_t kRowsPerPass = 256 / kLanesPerRow;
    constexpr uint32_t kPasses = kSwapRows / kRowsPerPass;
    const uint32_t cLocal = (threadIdx.x % kLanesPerRow) * kVec;
    const uint32_t rowInPass = threadIdx.x / kLanesPerRow;
    uint4 v[kPasses];
#pragma unroll
    for (uint32_t i = 0; i != kPasses; ++i) {
      const T *from = source(i * kRowsPerPass + rowInPass, c0 + cLocal);
      v[i] = from ? *reinterpret_cast<const uint4 *>(from) : uint4{0, 0, 0, 0};
    }
#pragma unroll
    for (uint32_t i = 0; i != kPasses; ++i) {
      const T *e = reinterpret_cast<const T *>(&v[i]);
#pragma unroll
      for (uint32_t k = 0; k != kVec; ++k)
        tile[i * kRowsPerPass + rowInPass][cLocal + k] = e[k];
    }
  } else {
    constexpr uint32_t kPasses = kSwapRows / 4;
    T v[kPasses];
#pragma unroll
    for (uint32_t i = 0; i != kPasses; ++i) {
      const T *from = source(i * 4 + wave, c0 + lane);
      v[i] = from ? *from : T(0);
    }
#pragma unroll
    for (uint32_t i = 0; i != kPasses; ++i)
      tile[i * 4 + wave][lane] = v[i];
  }
  __syncthreads();
  if (a.vectorStores) {
    // A thread gathers 16 bytes of consecutive batch entries of one channel
    // (consecutive rows of the tile); consecutive lanes take consecutive
    // such pieces, then the next channel.  The batch size and every stride
    // are multiples of the vector length.
    constexpr uint32_t kVec = 16 / sizeof(T);
    constexpr uint32_t kPieces = kSwapRows / kVec;
#pragma unroll 2
    for (uint32_t i = threadIdx.x; i < kSwapChans * kPieces; i += 256) {
      const uint32_t cLocal = i / kPieces, row = (i % kPieces) * kVec;
      const uint32_t p = p0 + row / a.batchPerTile;
      const uint32_t b = b0 + row % a.batchPerTile;
      const uint32_t c = c0 + cLocal;
      if (p < a.pixels && b < a.batch && c < a.chans) {
        union {
          uint4 raw;
          T e[kVec];
        } v;
#pragma unroll
        for (uint32_t k = 0; k != kVec; ++k)
          v.e[k] = T(tile[row + k][cLocal]);
        *reinterpret_cast<uint4 *>(dst + g * a.strideG + c * a.strideC +
                                   p * a.strideP + b) = v.raw;
      }
    }
    return;
  }
  // 64 lanes = 64 consecutive rows of the tile: consecutive batch entries,
  // then the next pixel.
#pragma unroll 4
  for (uint32_t i = wave; i < kSwapChans * 2; i += 4) {
    const uint32_t cLocal = i / 2, row = (i % 2) * 64 + lane;
    const uint32_t p = p0 + row / a.batchPerTile;
    const uint32_t b = b0 + row % a.batchPerTile;
    const uint32_t c = c0 + cLocal;
    if (p < a.pixels && b < a.batch && c < a.chans)
      dst[g * a.strideG + c * a.strideC + p * a.strideP + b] =
          T(tile[row][cLocal]);
  }
}

template <class T, bool VEC>
__global__ __launch_bounds__(256) void swapBatchChansKernel(
    SwapArgs a, const T *__restrict__ src, T *__restrict__ dst) {
  swapBatchChansTile<T, VEC>(a, src, dst, blockIdx.x, blockIdx.y, blockIdx.z);
}

/// Two such rearrangements in one launch (the two operands of a weight update
/// pass): the grid's z extent is the sum of theirs, x and y cover the larger;
/// workgroups outside their tensor's own grid have nothing to do.
struct SwapPairArgs {
  SwapArgs a[2];
  uint32_t gridX[2], gridY[2], gridZ0; // z blocks of the first
};
template <class T>
__global__ __launch_bounds__(256) void swapBatchChansPairKernel(
    SwapPairArgs m, const T *__restrict__ src0, T *__restrict__ dst0,
    const T *__restrict__ src1, T *__restrict__ dst1) {
  const uint32_t which = blockIdx.z < m.gridZ0 ? 0 : 1;
  if (blockIdx.x >= m.gridX[which] || blockIdx.y >= m.gridY[which])
    return;
  if (which == 0)
    swapBatchChansTile<T, true>(m.a[0], src0, dst0, blockIdx.x, blockIdx.y,
                                blockIdx.z);
  else
    swapBatchChansTile<T, true>(m.a[1], src1, dst1, blockIdx.x, blockIdx.y,
                                blockIdx.z - m.gridZ0);
}

template <class T>
__global__ __launch_bounds__(256) void zeroKernel(T *dst, uint64_t total) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid < total)
    dst[tid] = T(0);
}

constexpr uint32_t kReduceChans = 64, kReduceLanes = 4;

/// partial[split][c] = sum over the rows of `split` of z[row][c], fp32.
template <typename T>
__global__ __launch_bounds__(256) void channelSumKernel(
    const T *__restrict__ z, float *__restrict__ partial, uint64_t rows,
    uint64_t channels, uint64_t rowsPerSplit) {
  __shared__ float lanes[kReduceLanes][kReduceChans];
  const uint32_t cLocal = threadIdx.x % kReduceChans;
  const uint32_t lane = threadIdx.x / kReduceChans;
  const uint64_t c = uint64_t(blockIdx.x) * kReduceChans + cLocal;
  const uint64_t first = uint64_t(blockIdx.y) * rowsPerSplit;
  const uint64_t last = min(first + rowsPerSplit, rows);
  float sum = 0.f;
  if (c < channels)
    for (uint64_t r = first + lane; r < last; r += kReduceLanes)
      sum += Load<T>::at(z, r * channels + c, 0);
  lanes[lane][cLocal] = sum;
  __syncthreads();
  if (lane == 0 && c < channels) {
    float total = lanes[0][cLocal];
    for (uint32_t l = 1; l != kReduceLanes; ++l)
      total += lanes[l][cLocal];
    partial[uint64_t(blockIdx.y) * channels + c] = total;
  }
}

/// biases[c] += scale * sum over splits of partial[split][c], splits in order.
template <typename T>
__global__ __launch_bounds__(256) void biasUpdateKernel(
    T *biases, const float *__restrict__ partial, float scale,
    uint64_t channels, uint32_t splits) {
  const uint64_t c = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (c >= channels)
    return;
  float total = 0.f;
  for (uint32_t s = 0; s != splits; ++s)
    total += partial[uint64_t(s) * channels + c];
  storeOut(biases, c, Load<T>::at(biases, c, 0) + scale * total);
}

/// The other way round, for weight deltas: the f diagonal blocks of every
/// fused group of [G / f][f co][f ci][taps] -> [G][co][ci][taps].  One element
/// of the result per thread.
template <class T>
__global__ __launch_bounds__(256) void
unfuseGroupWeightsKernel(const T *__restrict__ src, T *__restrict__ dst,
                         uint64_t f, uint64_t co, uint64_t ci, uint64_t taps,
                         uint64_t total) {
  const uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total)
    return;
  const uint64_t tap = i % taps;
  uint64_t rest = i / taps;
  const uint64_t k = rest % ci;
  rest /= ci;
  const uint64_t n = rest % co;
  const uint64_t g = rest / co;
  const uint64_t fused = g / f, a = g % f;
  dst[i] = src[((fused * f * co + a * co + n) * (f * ci) + a * ci + k) * taps +
               tap];
}

/// Weights [G][co][ci][taps] of G conv groups -> [G / f][f co][f ci][taps] of
/// G / f groups that each take f of them as one: block (a, b) of a fused
/// group's f x f blocks of co x ci channels is group (f g' + a)'s weights
/// where a == b and zero elsewhere.  One element of the result per thread.
template <class T>
__global__ __launch_bounds__(256) void
fuseGroupWeightsKernel(const T *__restrict__ src, T *__restrict__ dst,
                       uint64_t f, uint64_t co, uint64_t ci, uint64_t taps,
                       uint64_t total) {
  const uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i >= total)
    return;
  const uint64_t tap = i % taps;
  uint64_t rest = i / taps;
  const uint64_t k = rest % (f * ci);
  rest /= f * ci;
  const uint64_t n = rest % (f * co);
  const uint64_t fused = rest / (f * co);
  const uint64_t a = n / co, b = k / ci;
  dst[i] = a == b ? src[(((fused * f + a) * co + n % co) * ci + k % ci) * taps +
                        tap]
                  : T(0);
}

} // namespace

hipError_t launchPermute4(const void *src, void *dst, const uint64_t srcDims[4],
                          const int perm[4], int elemBytes,
                          hipStream_t stream) {
  uint64_t srcStrides[4];
  srcStrides[3] = 1;
  for (int i = 2; i >= 0; --i)
    srcStrides[i] = srcStrides[i + 1] * srcDims[i + 1];
  PermuteArgs a;
  a.total = 1;
  for (int j = 0; j != 4; ++j) {
    a.dstDims[j] = srcDims[perm[j]];
    a.srcStride[j] = srcStrides[perm[j]];
    a.total *= a.dstDims[j];
  }
  if (a.total == 0)
    return hipSuccess;
  const uint64_t blocks = (a.total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  switch (elemBytes) {
  case 1:
    hipLaunchKernelGGL(permuteKernel<uint8_t>, grid, block, 0, stream, a,
                       static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst));
    break;
  case 2:
    hipLaunchKernelGGL(permuteKernel<uint16_t>, grid, block, 0, stream, a,
                       static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst));
    break;
  case 4:
    hipLaunchKernelGGL(permuteKernel<uint32_t>, grid, block, 0, stream, a,
                       static_cast<const uint32_t *>(src),
                       static_cast<uint32_t *>(dst));
    break;
  default:
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launchPackIgemmWeights(const void *src, void *dst, uint32_t groups,
                                  uint32_t co, uint32_t ci, uint32_t taps,
                                  uint32_t coPadded, uint32_t kPadded,
                                  int elemBytes, hipStream_t stream,
                                  bool chansTransposed, uint32_t ciPadded,
                                  const IgemmTapSelection *select) {
  const IgemmTapSelection chosen = select ? *select : IgemmTapSelection{};
  if (ciPadded == 0)
    ciPadded = ci;
  if (ciPadded < ci)
    return hipErrorInvalidValue;
  const uint64_t total = uint64_t(groups) * coPadded * kPadded;
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (elemBytes == 1)
    hipLaunchKernelGGL(packIgemmWeightsKernel<uint8_t>, grid, block, 0, stream,
                       static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst), co, ci, ciPadded, taps,
                       coPadded, kPadded, total, chansTransposed,
                       select != nullptr, chosen);
  else if (elemBytes == 2)
    hipLaunchKernelGGL(packIgemmWeightsKernel<uint16_t>, grid, block, 0, stream,
                       static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst), co, ci, ciPadded, taps,
                       coPadded, kPadded, total, chansTransposed,
                       select != nullptr, chosen);
  else if (elemBytes == 4)
    hipLaunchKernelGGL(packIgemmWeightsKernel<uint32_t>, grid, block, 0, stream,
                       static_cast<const uint32_t *>(src),
                       static_cast<uint32_t *>(dst), co, ci, ciPadded, taps,
                       coPadded, kPadded, total, chansTransposed,
                       select != nullptr, chosen);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launchPadChans(const void *src, void *dst, uint64_t pixels,
                          uint32_t groups, uint32_t ci, uint32_t ciPadded,
                          int elemBytes, hipStream_t stream) {
  if ((elemBytes != 1 && elemBytes != 2 && elemBytes != 4) || ciPadded < ci ||
      (uint64_t(ciPadded) * elemBytes) % 16 != 0)
    return hipErrorInvalidValue;
  const uint64_t vectors =
      pixels * groups * (uint64_t(ciPadded) * elemBytes / 16);
  if (vectors == 0)
    return hipSuccess;
  const uint64_t blocks = (vectors + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (elemBytes == 1)
    hipLaunchKernelGGL(padChansKernel<uint8_t>, grid, block, 0, stream,
                       static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst), vectors, ci, ciPadded);
  else if (elemBytes == 2)
    hipLaunchKernelGGL(padChansKernel<uint16_t>, grid, block, 0, stream,
                       static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst), vectors, ci, ciPadded);
  else
    hipLaunchKernelGGL(padChansKernel<uint32_t>, grid, block, 0, stream,
                       static_cast<const uint32_t *>(src),
                       static_cast<uint32_t *>(dst), vectors, ci, ciPadded);
  return hipGetLastError();
}

hipError_t launchWeightsTransposeChansFlipXY(const void *src, void *dst,
                                             uint64_t groups, uint64_t co,
                                             uint64_t ci, uint32_t numDims,
                                             const uint32_t *kernelShape,
                                             int elemBytes,
                                             hipStream_t stream) {
  if (numDims > uint32_t(kMaxDims))
    return hipErrorInvalidValue;
  FlipArgs a{};
  a.co = co, a.ci = ci, a.taps = 1, a.numDims = numDims;
  for (uint32_t d = 0; d != numDims; ++d) {
    a.shape[d] = kernelShape[d];
    a.taps *= kernelShape[d];
  }
  a.total = groups * co * ci * a.taps;
  if (a.total == 0)
    return hipSuccess;
  const uint64_t blocks = (a.total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (elemBytes == 1)
    hipLaunchKernelGGL(transposeChansFlipKernel<uint8_t>, grid, block, 0,
                       stream, a, static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst));
  else if (elemBytes == 2)
    hipLaunchKernelGGL(transposeChansFlipKernel<uint16_t>, grid, block, 0,
                       stream, a, static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst));
  else if (elemBytes == 4)
    hipLaunchKernelGGL(transposeChansFlipKernel<uint32_t>, grid, block, 0,
                       stream, a, static_cast<const uint32_t *>(src),
                       static_cast<uint32_t *>(dst));
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launchAddBias(int type, void *acts, const void *bias,
                         uint64_t outerElems, uint64_t channels,
                         hipStream_t stream) {
  const uint64_t total = outerElems * channels;
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (type == kFloat)
    hipLaunchKernelGGL(addBiasKernel<float>, grid, block, 0, stream,
                       static_cast<float *>(acts),
                       static_cast<const float *>(bias), total, channels);
  else if (type == kHalf)
    hipLaunchKernelGGL(addBiasKernel<__half>, grid, block, 0, stream,
                       static_cast<__half *>(acts),
                       static_cast<const __half *>(bias), total, channels);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

namespace {
struct SwapLaunch {
  SwapArgs a;
  dim3 grid;
  bool vectorLoads;
};

/// Tile shape, grid and vector widths of one rearrangement.
hipError_t prepareSwap(const void *src, const void *dst, uint32_t batch,
                       uint32_t pixels, uint32_t groups, uint32_t chans,
                       uint64_t strideG, uint64_t strideC, uint64_t strideP,
                       int elemBytes, SwapLaunch &l) {
  if (elemBytes != 2 && elemBytes != 4)
    return hipErrorInvalidValue;
  SwapArgs &a = l.a;
  a.batch = batch, a.pixels = pixels, a.groups = groups, a.chans = chans;
  // As much of the batch as a tile takes (a power of two, so that it divides
  // the 128 rows), the rest of the rows for neighbouring pixels.
  a.batchPerTile = 1;
  while (a.batchPerTile < kSwapRows && a.batchPerTile < batch)
    a.batchPerTile *= 2;
  a.pixelsPerTile = kSwapRows / a.batchPerTile;
  a.strideG = strideG, a.strideC = strideC, a.strideP = strideP;
  const uint64_t gx = uint64_t((chans + kSwapChans - 1) / kSwapChans) * groups;
  const uint64_t gy = (pixels + a.pixelsPerTile - 1) / a.pixelsPerTile;
  const uint64_t gz = (batch + a.batchPerTile - 1) / a.batchPerTile;
  if (gx > 0x7fffffffull || gy > 65535 || gz > 65535)
    return hipErrorInvalidConfiguration;
  l.grid = dim3{uint32_t(gx), uint32_t(gy), uint32_t(gz)};
  // 16-byte loads need every row of channels to start on a 16-byte boundary;
  // 16-byte stores, every run of batch entries.
  const uint32_t perVector = uint32_t(16 / elemBytes);
  l.vectorLoads = chans % perVector == 0 &&
                  reinterpret_cast<uintptr_t>(src) % 16 == 0;
  a.vectorStores = batch % perVector == 0 && a.batchPerTile >= perVector &&
                   strideG % perVector == 0 && strideC % perVector == 0 &&
                   strideP % perVector == 0 &&
                   reinterpret_cast<uintptr_t>(dst) % 16 == 0;
  return hipSuccess;
}
} // namespace

hipError_t launchSwapBatchChans(const void *src, void *dst, uint32_t batch,
                                uint32_t pixels, uint32_t groups,
                                uint32_t chans, uint64_t strideG,
                                uint64_t strideC, uint64_t strideP,
                                int elemBytes, hipStream_t stream) {
  if (uint64_t(batch) * pixels * groups * chans == 0)
    return hipSuccess;
  SwapLaunch l;
  const hipError_t e = prepareSwap(src, dst, batch, pixels, groups, chans,
                                   strideG, strideC, strideP, elemBytes, l);
  if (e != hipSuccess)
    return e;
  const SwapArgs &a = l.a;
  const dim3 grid = l.grid, block{256};
  const bool vec = l.vectorLoads;
  if (elemBytes == 2) {
    const auto *from = static_cast<const uint16_t *>(src);
    auto *to = static_cast<uint16_t *>(dst);
    if (vec)
      hipLaunchKernelGGL((swapBatchChansKernel<uint16_t, true>), grid, block, 0,
                         stream, a, from, to);
    else
      hipLaunchKernelGGL((swapBatchChansKernel<uint16_t, false>), grid, block,
                         0, stream, a, from, to);
  } else {
    const auto *from = static_cast<const uint32_t *>(src);
    auto *to = static_cast<uint32_t *>(dst);
    if (vec)
      hipLaunchKernelGGL((swapBatchChansKernel<uint32_t, true>), grid, block, 0,
                         stream, a, from, to);
    else
      hipLaunchKernelGGL((swapBatchChansKernel<uint32_t, false>), grid, block,
                         0, stream, a, from, to);
  }
  return hipGetLastError();
}

hipError_t launchSwapBatchChansPair(const SwapBatchChans &first,
                                    const SwapBatchChans &second,
                                    int elemBytes, hipStream_t stream) {
  auto alone = [&](const SwapBatchChans &x) {
    return launchSwapBatchChans(x.src, x.dst, x.batch, x.pixels, x.groups,
                                x.chans, x.strideG, x.strideC, x.strideP,
                                elemBytes, stream);
  };
  auto empty = [](const SwapBatchChans &x) {
    return uint64_t(x.batch) * x.pixels * x.groups * x.chans == 0;
  };
  SwapLaunch l[2];
  bool together = !empty(first) && !empty(second);
  if (together) {
    const SwapBatchChans *both[2] = {&first, &second};
    for (int i = 0; i != 2 && together; ++i) {
      const SwapBatchChans &x = *both[i];
      together = prepareSwap(x.src, x.dst, x.batch, x.pixels, x.groups,
                             x.chans, x.strideG, x.strideC, x.strideP,
                             elemBytes, l[i]) == hipSuccess &&
                 l[i].vectorLoads;
    }
    together = together && l[0].grid.z + l[1].grid.z <= 65535;
  }
  if (!together) {
    const hipError_t e = alone(first);
    return e != hipSuccess ? e : alone(second);
  }
  SwapPairArgs m;
  for (int i = 0; i != 2; ++i)
    m.a[i] = l[i].a, m.gridX[i] = l[i].grid.x, m.gridY[i] = l[i].grid.y;
  m.gridZ0 = l[0].grid.z;
  const dim3 grid{l[0].grid.x > l[1].grid.x ? l[0].grid.x : l[1].grid.x,
                  l[0].grid.y > l[1].grid.y ? l[0].grid.y : l[1].grid.y,
                  l[0].grid.z + l[1].grid.z};
  if (elemBytes == 2)
    hipLaunchKernelGGL(swapBatchChansPairKernel<uint16_t>, grid, dim3{256}, 0,
                       stream, m, static_cast<const uint16_t *>(first.src),
                       static_cast<uint16_t *>(first.dst),
                       static_cast<const uint16_t *>(second.src),
                       static_cast<uint16_t *>(second.dst));
  else
    hipLaunchKernelGGL(swapBatchChansPairKernel<uint32_t>, grid, dim3{256}, 0,
                       stream, m, static_cast<const uint32_t *>(first.src),
                       static_cast<uint32_t *>(first.dst),
                       static_cast<const uint32_t *>(second.src),
                       static_cast<uint32_t *>(second.dst));
  return hipGetLastError();
}

hipError_t launchZero(void *dst, uint64_t bytes, hipStream_t stream) {
  if (bytes == 0)
    return hipSuccess;
  if (bytes % 4 != 0)
    return hipErrorInvalidValue;
  const uint64_t total = bytes / 4, blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(zeroKernel<uint32_t>, dim3(uint32_t(blocks)), dim3(256), 0,
                     stream, static_cast<uint32_t *>(dst), total);
  return hipGetLastError();
}

namespace {
/// One element of the padded output field per thread; those inside the
/// convolution's own outputs are left alone.
template <class T>
__global__ __launch_bounds__(256) void fillOutputPaddingKernel(
    T *__restrict__ out, const T *__restrict__ bias, uint64_t total,
    uint32_t fullD, uint32_t fullH, uint32_t fullW, uint32_t offD,
    uint32_t offH, uint32_t offW, uint32_t insideD, uint32_t insideH,
    uint32_t insideW, uint32_t chans) {
  const uint64_t tid = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (tid >= total)
    return;
  const uint64_t pixel = tid / chans;
  const uint32_t c = uint32_t(tid - pixel * chans);
  const uint32_t w = uint32_t(pixel % fullW);
  const uint32_t h = uint32_t((pixel / fullW) % fullH);
  const uint32_t z = uint32_t((pixel / fullW / fullH) % fullD);
  if (z - offD < insideD && h - offH < insideH && w - offW < insideW)
    return;
  out[tid] = bias ? bias[c] : T(0);
}
} // namespace

namespace {
/// The same with one 16-byte vector per thread and 32-bit arithmetic inside
/// an image (blockIdx.y, .z: the image); channel counts that are whole
/// vectors.
template <class T>
__global__ __launch_bounds__(256) void fillOutputPaddingVectorKernel(
    T *__restrict__ out, const T *__restrict__ bias, uint32_t imageVectors,
    uint32_t fullH, uint32_t fullW, uint32_t offD, uint32_t offH,
    uint32_t offW, uint32_t insideD, uint32_t insideH, uint32_t insideW,
    uint32_t vecsPerPixel) {
  constexpr uint32_t kVec = 16 / sizeof(T);
  const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= imageVectors)
    return;
  const uint32_t pixel = idx / vecsPerPixel, vec = idx - pixel * vecsPerPixel;
  const uint32_t row = pixel / fullW, w = pixel - row * fullW;
  const uint32_t z = row / fullH, h = row - z * fullH;
  if (z - offD < insideD && h - offH < insideH && w - offW < insideW)
    return;
  const uint64_t image = uint64_t(blockIdx.z) * gridDim.y + blockIdx.y;
  uint4 v{0, 0, 0, 0};
  if (bias)
    v = *reinterpret_cast<const uint4 *>(bias + vec * kVec);
  reinterpret_cast<uint4 *>(out)[image * imageVectors + idx] = v;
}
} // namespace

hipError_t launchFillOutputPadding(int type, void *out, const void *bias,
                                   uint64_t images, uint32_t fullD,
                                   uint32_t fullH, uint32_t fullW,
                                   uint32_t offD, uint32_t offH,
                                   uint32_t offW, uint32_t insideD,
                                   uint32_t insideH, uint32_t insideW,
                                   uint32_t chans, hipStream_t stream) {
  const uint64_t total = images * fullD * fullH * fullW * chans;
  if (total == 0)
    return hipSuccess;
  const uint32_t vecElems = type == kHalf ? 8 : 4;
  const uint64_t imageVectors =
      uint64_t(fullD) * fullH * fullW * (chans / vecElems);
  if ((type == kHalf || type == kFloat) && chans % vecElems == 0 &&
      imageVectors < (1ull << 31) &&
      (bias == nullptr || reinterpret_cast<uintptr_t>(bias) % 16 == 0) &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    // images as grid y (and z beyond 32768 of them)
    const uint32_t gy = uint32_t(images < 32768 ? images : 32768);
    if (images % gy == 0 && images / gy < 65536) {
      const dim3 grid{uint32_t((imageVectors + 255) / 256), gy,
                      uint32_t(images / gy)};
      if (type == kHalf)
        hipLaunchKernelGGL(fillOutputPaddingVectorKernel<__half>, grid,
                           dim3(256), 0, stream, static_cast<__half *>(out),
                           static_cast<const __half *>(bias),
                           uint32_t(imageVectors), fullH, fullW, offD, offH,
                           offW, insideD, insideH, insideW, chans / vecElems);
      else
        hipLaunchKernelGGL(fillOutputPaddingVectorKernel<float>, grid,
                           dim3(256), 0, stream, static_cast<float *>(out),
                           static_cast<const float *>(bias),
                           uint32_t(imageVectors), fullH, fullW, offD, offH,
                           offW, insideD, insideH, insideW, chans / vecElems);
      return hipGetLastError();
    }
  }
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  if (type == kHalf)
    hipLaunchKernelGGL(fillOutputPaddingKernel<__half>, dim3(uint32_t(blocks)),
                       dim3(256), 0, stream, static_cast<__half *>(out),
                       static_cast<const __half *>(bias), total, fullD, fullH,
                       fullW, offD, offH, offW, insideD, insideH, insideW,
                       chans);
  else if (type == kFloat)
    hipLaunchKernelGGL(fillOutputPaddingKernel<float>, dim3(uint32_t(blocks)),
                       dim3(256), 0, stream, static_cast<float *>(out),
                       static_cast<const float *>(bias), total, fullD, fullH,
                       fullW, offD, offH, offW, insideD, insideH, insideW,
                       chans);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

uint32_t biasUpdateSplits(uint64_t rows) {
  const uint64_t splits = (rows + 127) / 128;
  return uint32_t(splits < 1 ? 1 : splits > 256 ? 256 : splits);
}

size_t biasUpdateWorkspaceBytes(uint64_t rows, uint64_t channels) {
  return size_t(biasUpdateSplits(rows)) * channels * sizeof(float);
}

hipError_t launchBiasUpdate(int deltasType, const void *zDeltas, uint64_t rows,
                            uint64_t channels, int biasType, void *biases,
                            float scale, void *workspace, hipStream_t stream) {
  if (channels == 0)
    return hipSuccess;
  const uint32_t splits = biasUpdateSplits(rows);
  const uint64_t rowsPerSplit = (rows + splits - 1) / splits;
  const uint64_t chanBlocks = (channels + kReduceChans - 1) / kReduceChans;
  if (chanBlocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  float *partial = static_cast<float *>(workspace);
  const dim3 grid{uint32_t(chanBlocks), splits}, block{256};
  if (deltasType == kFloat)
    hipLaunchKernelGGL(channelSumKernel<float>, grid, block, 0, stream,
                       static_cast<const float *>(zDeltas), partial, rows,
                       channels, rowsPerSplit);
  else if (deltasType == kHalf)
    hipLaunchKernelGGL(channelSumKernel<__half>, grid, block, 0, stream,
                       static_cast<const __half *>(zDeltas), partial, rows,
                       channels, rowsPerSplit);
  else
    return hipErrorInvalidValue;
  const dim3 grid2{uint32_t((channels + 255) / 256)};
  if (biasType == kFloat)
    hipLaunchKernelGGL(biasUpdateKernel<float>, grid2, block, 0, stream,
                       static_cast<float *>(biases), partial, scale, channels,
                       splits);
  else if (biasType == kHalf)
    hipLaunchKernelGGL(biasUpdateKernel<__half>, grid2, block, 0, stream,
                       static_cast<__half *>(biases), partial, scale, channels,
                       splits);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launchUnfuseGroupWeights(const void *src, void *dst,
                                    uint64_t groups, uint64_t perGroup,
                                    uint64_t co, uint64_t ci, uint64_t taps,
                                    int elemBytes, hipStream_t stream) {
  const uint64_t total = groups * co * ci * taps;
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull || groups % perGroup != 0)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (elemBytes == 4)
    hipLaunchKernelGGL(unfuseGroupWeightsKernel<uint32_t>, grid, block, 0,
                       stream, static_cast<const uint32_t *>(src),
                       static_cast<uint32_t *>(dst), perGroup, co, ci, taps,
                       total);
  else if (elemBytes == 2)
    hipLaunchKernelGGL(unfuseGroupWeightsKernel<uint16_t>, grid, block, 0,
                       stream, static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst), perGroup, co, ci, taps,
                       total);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launchFuseGroupWeights(const void *src, void *dst, uint64_t groups,
                                  uint64_t perGroup, uint64_t co, uint64_t ci,
                                  uint64_t taps, int elemBytes,
                                  hipStream_t stream) {
  const uint64_t total = groups * perGroup * co * ci * taps;
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull || groups % perGroup != 0)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (elemBytes == 4)
    hipLaunchKernelGGL(fuseGroupWeightsKernel<uint32_t>, grid, block, 0, stream,
                       static_cast<const uint32_t *>(src),
                       static_cast<uint32_t *>(dst), perGroup, co, ci, taps,
                       total);
  else if (elemBytes == 2)
    hipLaunchKernelGGL(fuseGroupWeightsKernel<uint16_t>, grid, block, 0, stream,
                       static_cast<const uint16_t *>(src),
                       static_cast<uint16_t *>(dst), perGroup, co, ci, taps,
                       total);
  else if (elemBytes == 1)
    hipLaunchKernelGGL(fuseGroupWeightsKernel<uint8_t>, grid, block, 0, stream,
                       static_cast<const uint8_t *>(src),
                       static_cast<uint8_t *>(dst), perGroup, co, ci, taps,
                       total);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launchScaledAdd(int type, void *a, float scaleA, const void *b,
                           float scaleB, uint64_t total, hipStream_t stream) {
  if (total == 0)
    return hipSuccess;
  const uint64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const dim3 grid{uint32_t(blocks)}, block{256};
  if (type == kFloat)
    hipLaunchKernelGGL(scaledAddKernel<float>, grid, block, 0, stream,
                       static_cast<float *>(a), scaleA,
                       static_cast<const float *>(b), scaleB, total);
  else if (type == kHalf)
    hipLaunchKernelGGL(scaledAddKernel<__half>, grid, block, 0, stream,
                       static_cast<__half *>(a), scaleA,
                       static_cast<const __half *>(b), scaleB, total);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

} // namespace mxk

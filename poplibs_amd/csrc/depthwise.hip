// Depthwise forward convolution (one input and one output channel per group):
// the memory-bound case PopLibs serves with its HorizontalMac vertices
// (lib/poplin/codelets/ConvPartialHorizontalMac.cpp:34-133).  No matrix cores:
// at 1.8 flop per byte the only thing that matters is to move every input
// element from HBM once, write every output once, and keep enough bytes in
// flight to cover HBM latency.
//
// Channels-last layout; the unit of work is a 16-byte vector of 8 consecutive
// fp16 channels.  A workgroup produces a tile of tileH x tileW output pixels
// for a block of up to 16 channel vectors:
//   1. all of the input patch the tile needs ((tileH-1)*strideH +
//      (kH-1)*dilH + 1 rows, likewise columns) is requested at once with
//      16-byte buffer loads that write straight into LDS - one burst per
//      workgroup, the deepest memory-level parallelism the hardware offers,
//      no staging registers.  Patch elements that fall on padding get an
//      out-of-range offset, for which the buffer unit delivers zeros, so the
//      compute loop has no bounds checks;
//   2. after one barrier each thread forms its outputs from LDS:
//      products and sums in fp32 (v_fma_mix_f32 on the packed halves);
//   3. 16-byte (fp16 output) or 2 x 16-byte (fp32 output) coalesced stores.
// Several workgroups share a CU (the patch is kept under 52 KB of the 160 KB
// LDS), so one workgroup's loads overlap another's arithmetic and stores.
// Neighbouring tiles overlap by the kernel halo; workgroups are numbered so
// that each XCD walks a contiguous run of tiles and the halo re-reads hit its
// own L2 instead of HBM.
#include "device_types.hpp"
#include "kernels.hpp"

namespace mxk {
namespace {

constexpr int kThreads = 256;
constexpr uint32_t kOutOfRange = 0x80000000u;

using LdsPtr = __attribute__((address_space(3))) void *;

__device__ __forceinline__ uint32_t xcdSwizzle(uint32_t bid, uint32_t total) {
  const uint32_t xcd = bid & 7u, idx = bid >> 3;
  const uint32_t q = total >> 3, rem = total & 7u;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

/// 16 bytes per lane from a buffer straight into LDS: lane l's data lands at
/// dst + 16 l (dst is wave-uniform); out-of-range offsets deliver zeros.  The
/// builtin exists for the GPU target only; the host pass sees an empty body.
__device__ __forceinline__ void loadToLds(__amdgpu_buffer_rsrc_t buffer,
                                          LdsPtr dst, uint32_t vectorOffset) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(buffer, dst, 16, vectorOffset, 0, 0,
                                           0);
#endif
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
      o.h2[i] = roundPairToHalf(v[2 * i], v[2 * i + 1]);
    *reinterpret_cast<uint4 *>(p) = o.raw;
  }
};
template <> struct StoreVec<float> {
  static __device__ __forceinline__ void put(float *p, const float (&v)[8]) {
    *reinterpret_cast<float4 *>(p) = float4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4 *>(p + 4) = float4{v[4], v[5], v[6], v[7]};
  }
};

/// A 16-byte vector of E channels of the input type as fp32 (fp8: `format`
/// as in decodeFp8).
template <class InT> struct InVec;
template <> struct InVec<__half> {
  static constexpr int E = 8;
  static __device__ __forceinline__ void unpack(const uint4 &raw, int,
                                                float (&f)[8]) {
    Vec8 v;
    v.raw = raw;
#pragma unroll
    for (int i = 0; i != 4; ++i) {
      const float2 two = __half22float2(v.h2[i]);
      f[2 * i] = two.x, f[2 * i + 1] = two.y;
    }
  }
};
template <> struct InVec<float> {
  static constexpr int E = 4;
  static __device__ __forceinline__ void unpack(const uint4 &raw, int,
                                                float (&f)[4]) {
    f[0] = __uint_as_float(raw.x), f[1] = __uint_as_float(raw.y);
    f[2] = __uint_as_float(raw.z), f[3] = __uint_as_float(raw.w);
  }
};
template <> struct InVec<uint8_t> {
  static constexpr int E = 16;
  static __device__ __forceinline__ void unpack(const uint4 &raw, int format,
                                                float (&f)[16]) {
    // (the hardware's conversions of OCP E4M3 / E5M2 pairs: the decoding in
    // software costs the kernel a factor of ten)
    const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#if defined(__HIP_DEVICE_COMPILE__)
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    if (format == 1) {
#pragma unroll
      for (int i = 0; i != 4; ++i) {
        const floatx2 lo =
            __builtin_amdgcn_cvt_pk_f32_fp8(int(words[i]), false);
        const floatx2 hi = __builtin_amdgcn_cvt_pk_f32_fp8(int(words[i]), true);
        f[4 * i] = lo.x, f[4 * i + 1] = lo.y;
        f[4 * i + 2] = hi.x, f[4 * i + 3] = hi.y;
      }
    } else {
#pragma unroll
      for (int i = 0; i != 4; ++i) {
        const floatx2 lo =
            __builtin_amdgcn_cvt_pk_f32_bf8(int(words[i]), false);
        const floatx2 hi = __builtin_amdgcn_cvt_pk_f32_bf8(int(words[i]), true);
        f[4 * i] = lo.x, f[4 * i + 1] = lo.y;
        f[4 * i + 2] = hi.x, f[4 * i + 3] = hi.y;
      }
    }
#else
    for (int i = 0; i != 16; ++i)
      f[i] = 0.0f * float(words[i / 4]) * float(format);
#endif
  }
};

/// E consecutive channels of the output.
template <class OutT, int E>
__device__ __forceinline__ void putVec(OutT *p, const float (&v)[E]) {
  if constexpr (E == 8) {
    StoreVec<OutT>::put(p, v);
  } else if constexpr (sizeof(OutT) == 4) {
#pragma unroll
    for (int i = 0; i != E; i += 4)
      *reinterpret_cast<float4 *>(p + i) =
          float4{v[i], v[i + 1], v[i + 2], v[i + 3]};
  } else if constexpr (E == 4) {
    const __half2 lo = roundPairToHalf(v[0], v[1]),
                  hi = roundPairToHalf(v[2], v[3]);
    *reinterpret_cast<uint2 *>(p) = uint2{__builtin_bit_cast(uint32_t, lo),
                                          __builtin_bit_cast(uint32_t, hi)};
  } else {
    static_assert(E == 16, "vectors of 4, 8 or 16 channels");
#pragma unroll
    for (int h = 0; h != 2; ++h) {
      Vec8 o;
#pragma unroll
      for (int i = 0; i != 4; ++i)
        o.h2[i] = roundPairToHalf(v[8 * h + 2 * i], v[8 * h + 2 * i + 1]);
      *reinterpret_cast<uint4 *>(p + 8 * h) = o.raw;
    }
  }
}

struct DwArgs {
  DepthwiseDesc d;
  // fp8 inputs: the tensors' formats (as decodeFp8 takes them) and
  // 2^(scaleIn + scaleWeights), applied to the sums before the bias
  int formatIn, formatWeights;
  float scale;
  uint32_t vecs;      // channels in 16-byte vectors (of 4, 8 or 16)
  uint32_t vecBlock;  // channel vectors per workgroup: vecs if <= 16, else 16
  uint32_t vecShift;  // log2(vecBlock) when the channels are split in blocks
  uint32_t vecBlocks; // ceil(vecs / vecBlock)
  uint32_t tilesH, tilesW;
  uint32_t patchH, patchW;
  uint32_t rowElems;  // patchW * vecBlock: 16-byte elements per patch row
  uint32_t rowPitch;  // rowElems rounded up to a multiple of 64
  // Compute phase: pixelsPerRound * vecBlock threads are active; a thread
  // keeps its channel vector and steps pixelsPerRound pixels per round.
  uint32_t pixelsPerRound, stepY, stepX; // pixelsPerRound = stepY*tileW+stepX
  uint32_t inBytes;
};

/// KH, KW > 0: kernel extents known at compile time (taps fully unrolled);
/// 0: taken from the descriptor.
/// PX > 0 (unit stride and dilation, KH and KW known): a thread forms PX
/// neighbouring output pixels of a row at once - for large kernels, where the
/// multiply-adds, not the bytes, are what a layer costs (7 x 7: 49 per
/// output) and a pixel at a time spends an LDS read and a tap load on every
/// one of them.  Per kernel row the thread reads the row's KW taps (kept in
/// LDS behind the patch, one copy per workgroup) and the PX + KW - 1 input
/// vectors under them once and multiplies PX x KW times: 13 multiply-adds per
/// 16-byte LDS read at 7 x 7 and PX = 7, against one.
/// InT: __half, float or uint8_t (fp8) inputs; the strips are for half.
template <int KH, int KW, class OutT, int PX = 0, class InT = __half>
__global__ __launch_bounds__(kThreads) void depthwiseKernel(
    DwArgs a, const InT *__restrict__ in, const InT *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out) {
  constexpr int E = InVec<InT>::E; // channels of a 16-byte vector
  static_assert(PX == 0 || E == 8, "strips: half inputs");
  extern __shared__ __align__(16) char lds[]; // patchH * rowPitch * 16 bytes
  const DepthwiseDesc &d = a.d;
  const uint32_t kH = KH ? KH : d.kH, kW = KW ? KW : d.kW;

  uint32_t tile = xcdSwizzle(blockIdx.x, gridDim.x);
  const uint32_t cb = tile % a.vecBlocks;
  tile /= a.vecBlocks;
  const uint32_t tw = tile % a.tilesW;
  tile /= a.tilesW;
  const uint32_t th = tile % a.tilesH;
  const uint32_t b = tile / a.tilesH;

  const uint32_t oh0 = th * d.tileH, ow0 = tw * d.tileW;
  const uint32_t cv0 = cb * a.vecBlock;
  const uint32_t nvec = min(a.vecBlock, a.vecs - cv0); // vectors in this block
  const int ih0 = int(oh0 * d.strideH) - d.padH; // patch origin in the input
  const int iw0 = int(ow0 * d.strideW) - d.padW;

  // 1. the whole patch, one burst.  LDS holds patch row ph at byte
  // 16 * ph * rowPitch, element j = pw * vecBlock + v of the row at + 16 j; a
  // wave-wide load covers 64 consecutive j of one row.  No division: with all
  // channels in one block the row is contiguous in memory as well, otherwise
  // vecBlock is 16 and (pw, v) are a shift and a mask of j.
  const __amdgpu_buffer_rsrc_t inBuf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<InT *>(in), short(0), int(a.inBytes), 0x00020000);
  const uint32_t pixelBytes = d.channels * sizeof(InT);
  const uint32_t imageOff = b * d.inH * d.inW * pixelBytes;
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const uint32_t chunksPerRow = a.rowPitch >> 6;
  const uint32_t chunks = a.patchH * chunksPerRow;
  // Wave w takes 64-element chunks w, w + 4, ...; (ph, chunk in row) advance
  // without dividing.
  uint32_t ph = 0, cr = wave;
  while (cr >= chunksPerRow) {
    cr -= chunksPerRow;
    ++ph;
  }
  for (uint32_t chunk = wave; chunk < chunks; chunk += kThreads / 64) {
    const uint32_t j = cr * 64 + lane;
    uint32_t pw, v;
    if (a.vecBlocks == 1) {
      pw = 0; // row-contiguous: the offset below uses j directly
      v = j;
    } else {
      pw = j >> a.vecShift;
      v = j & (a.vecBlock - 1);
    }
    const int ih = ih0 + int(ph);
    bool ok = j < a.rowElems && ih >= int(d.loH) && ih < int(d.hiH);
    uint32_t off = imageOff + uint32_t(ih) * d.inW * pixelBytes;
    if (a.vecBlocks == 1) {
      // valid columns [loW, hiW) as a range of j
      const int jLo = (int(d.loW) - iw0) * int(a.vecBlock);
      const int jHi = (int(d.hiW) - iw0) * int(a.vecBlock);
      ok = ok && int(j) >= jLo && int(j) < jHi;
      off += uint32_t(iw0) * pixelBytes + j * 16;
    } else {
      const int iw = iw0 + int(pw);
      ok = ok && iw >= int(d.loW) && iw < int(d.hiW) && v < nvec;
      off += uint32_t(iw) * pixelBytes + (cv0 + v) * 16;
    }
    loadToLds(inBuf, (LdsPtr)(lds + (ph * a.rowPitch + cr * 64) * 16),
              ok ? off : kOutOfRange);
    cr += kThreads / 64;
    while (cr >= chunksPerRow) {
      cr -= chunksPerRow;
      ++ph;
    }
  }

  // This thread's channel vector and first pixel; its kernel taps (3x3:
  // kept in registers for all its pixels).
  const uint32_t v = threadIdx.x % a.vecBlock;
  uint32_t p = threadIdx.x / a.vecBlock;
  const bool active = p < a.pixelsPerRound && v < nvec;
  const uint32_t c = (cv0 + (v < nvec ? v : 0)) * E;
  const InT *wC = w + c;
  constexpr bool kTapsInRegs = KH * KW != 0 && KH * KW <= 9;
  Vec8 taps[kTapsInRegs ? KH * KW : 1];
  if constexpr (kTapsInRegs) {
#pragma unroll
    for (int tap = 0; tap != KH * KW; ++tap)
      taps[tap].raw =
          *reinterpret_cast<const uint4 *>(wC + tap * d.channels);
  }
  float biasV[E];
#pragma unroll
  for (int i = 0; i != E; ++i)
    biasV[i] = bias ? Load<OutT>::at(bias, c + i, 0) : 0.0f;

  if constexpr (PX != 0) {
    static_assert(KH != 0 && KW != 0, "strips want the kernel's extents");
    // the taps, [tap][vecBlock] behind the patch
    uint4 *tapsLds =
        reinterpret_cast<uint4 *>(lds + a.patchH * a.rowPitch * 16);
    for (uint32_t i = threadIdx.x; i < KH * KW * a.vecBlock; i += kThreads) {
      const uint32_t tap = i / a.vecBlock, tv = i - tap * a.vecBlock;
      tapsLds[i] = *reinterpret_cast<const uint4 *>(
          w + tap * d.channels + (cv0 + (tv < nvec ? tv : 0)) * 8);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's loads landed
    __syncthreads();
    const uint32_t strips = (d.tileW + PX - 1) / PX;
    const uint32_t items = d.tileH * strips * a.vecBlock;
    const uint32_t owEnd = min(d.outW, ow0 + d.tileW);
    for (uint32_t item = threadIdx.x; item < items; item += kThreads) {
      const uint32_t iv = item % a.vecBlock, rest = item / a.vecBlock;
      const uint32_t sy = rest / strips, sx = (rest - sy * strips) * PX;
      const uint32_t oh = oh0 + sy;
      if (iv >= nvec || oh >= d.outH || ow0 + sx >= owEnd)
        continue;
      const uint32_t ic = (cv0 + iv) * 8;
      float acc[PX][8];
#pragma unroll
      for (int px = 0; px != PX; ++px)
#pragma unroll
        for (int i = 0; i != 8; ++i)
          acc[px][i] = bias ? Load<OutT>::at(bias, ic + i, 0) : 0.0f;
      const char *rowAt = lds + (sy * a.rowPitch + sx * a.vecBlock + iv) * 16;
      // (a kernel row at a time: unrolled over the rows the compiler asks for
      // every row's taps and inputs at once, 560 registers)
#pragma unroll 1
      for (int kh = 0; kh != KH; ++kh) {
        Vec8 k[KW], x[PX + KW - 1];
#pragma unroll
        for (int kw = 0; kw != KW; ++kw)
          k[kw].raw = tapsLds[(kh * KW + kw) * a.vecBlock + iv];
        // (a strip that ends beyond the tile reads on into the row's padding
        // or the next row - inside the LDS - for pixels that are not stored)
#pragma unroll
        for (int j = 0; j != PX + KW - 1; ++j)
          x[j].raw = *reinterpret_cast<const uint4 *>(rowAt +
                                                      j * a.vecBlock * 16);
#pragma unroll
        for (int px = 0; px != PX; ++px)
#pragma unroll
          for (int kw = 0; kw != KW; ++kw)
#pragma unroll
            for (int i = 0; i != 4; ++i) {
              const float2 xf = __half22float2(x[px + kw].h2[i]);
              const float2 kf = __half22float2(k[kw].h2[i]);
              acc[px][2 * i] = fmaf(xf.x, kf.x, acc[px][2 * i]);
              acc[px][2 * i + 1] = fmaf(xf.y, kf.y, acc[px][2 * i + 1]);
            }
        rowAt += a.rowPitch * 16;
      }
      OutT *to = out +
                 ((size_t(b) * d.outH + oh) * d.outW + ow0 + sx) * d.channels +
                 ic;
#pragma unroll
      for (int px = 0; px != PX; ++px)
        if (ow0 + sx + px < owEnd)
          StoreVec<OutT>::put(to + size_t(px) * d.channels, acc[px]);
    }
    return;
  }

  __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): this wave's loads landed
  __syncthreads();

  // 2. + 3.  One item = one output pixel x one channel vector.
  uint32_t ty = 0, tx = p;
  while (tx >= d.tileW) {
    tx -= d.tileW;
    ++ty;
  }
  const uint32_t pixels = d.tileH * d.tileW;
  if (active)
    for (; p < pixels; p += a.pixelsPerRound) {
      const uint32_t oh = oh0 + ty, ow = ow0 + tx;
      if (oh < d.outH && ow < d.outW) {
        float acc[E];
#pragma unroll
        for (int i = 0; i != E; ++i)
          acc[i] = E == 8 ? biasV[i] : 0.0f;
        const char *patch =
            lds + (ty * d.strideH * a.rowPitch +
                   tx * d.strideW * a.vecBlock + v) *
                      16;
#pragma unroll
        for (uint32_t kh = 0; kh < kH; ++kh)
#pragma unroll
          for (uint32_t kw = 0; kw < kW; ++kw) {
            Vec8 x, k;
            x.raw = *reinterpret_cast<const uint4 *>(
                patch +
                (kh * d.dilH * a.rowPitch + kw * d.dilW * a.vecBlock) * 16);
            if constexpr (kTapsInRegs)
              k = taps[kh * KW + kw];
            else
              k.raw = *reinterpret_cast<const uint4 *>(
                  wC + (kh * kW + kw) * d.channels);
            if constexpr (E == 8) {
#pragma unroll
              for (int i = 0; i != 4; ++i) {
                const float2 xf = __half22float2(x.h2[i]);
                const float2 kf = __half22float2(k.h2[i]);
                acc[2 * i] = fmaf(xf.x, kf.x, acc[2 * i]);
                acc[2 * i + 1] = fmaf(xf.y, kf.y, acc[2 * i + 1]);
              }
            } else {
              float xf[E], kf[E];
              InVec<InT>::unpack(x.raw, a.formatIn, xf);
              InVec<InT>::unpack(k.raw, a.formatWeights, kf);
#pragma unroll
              for (int i = 0; i != E; ++i)
                acc[i] = fmaf(xf[i], kf[i], acc[i]);
            }
          }
        if constexpr (E != 8) {
          // (fp8: the scale on the sum, then the bias)
#pragma unroll
          for (int i = 0; i != E; ++i)
            acc[i] = (E == 16 ? acc[i] * a.scale : acc[i]) + biasV[i];
        }
        putVec<OutT, E>(
            out + ((size_t(b) * d.outH + oh) * d.outW + ow) * d.channels + c,
            acc);
      }
      ty += a.stepY;
      tx += a.stepX;
      if (tx >= d.tileW) {
        tx -= d.tileW;
        ++ty;
      }
    }
}

constexpr uint32_t kLdsMost = kDepthwiseTileLdsMost;

template <int KH, int KW, class OutT, int PX = 0, class InT = __half>
hipError_t run(const DwArgs &a, uint32_t blocks, uint32_t ldsBytes,
               const void *in, const void *w, const void *bias, void *out,
               hipStream_t stream) {
  // (strips: the taps behind the patch)
  ldsBytes += PX ? KH * KW * a.vecBlock * 16 : 0;
  if (ldsBytes > kLdsMost)
    return hipErrorInvalidConfiguration;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void *>(
          &depthwiseKernel<KH, KW, OutT, PX, InT>),
      hipFuncAttributeMaxDynamicSharedMemorySize, kLdsMost);
  if (attr != hipSuccess)
    return attr;
  hipLaunchKernelGGL((depthwiseKernel<KH, KW, OutT, PX, InT>), dim3(blocks),
                     dim3(kThreads), ldsBytes, stream, a,
                     static_cast<const InT *>(in),
                     static_cast<const InT *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out));
  return hipGetLastError();
}

/// float or fp8 inputs: the kernel a pixel at a time, 3 x 3 taps unrolled.
template <class OutT, class InT>
hipError_t runOtherType(const DwArgs &a, uint32_t blocks, uint32_t ldsBytes,
                        const void *in, const void *w, const void *bias,
                        void *out, hipStream_t stream) {
  if (a.d.kH == 3 && a.d.kW == 3)
    return run<3, 3, OutT, 0, InT>(a, blocks, ldsBytes, in, w, bias, out,
                                   stream);
  return run<0, 0, OutT, 0, InT>(a, blocks, ldsBytes, in, w, bias, out,
                                 stream);
}

template <class OutT>
hipError_t runKernelShape(const DwArgs &a, uint32_t blocks, uint32_t ldsBytes,
                          const void *in, const void *w, const void *bias,
                          void *out, hipStream_t stream) {
  if (a.d.kH == 3 && a.d.kW == 3)
    return run<3, 3, OutT>(a, blocks, ldsBytes, in, w, bias, out, stream);
  const bool unit = a.d.strideH == 1 && a.d.strideW == 1 && a.d.dilH == 1 &&
                    a.d.dilW == 1;
  if (a.d.kH == 7 && a.d.kW == 7 && unit && a.d.stripPixels == 7)
    return run<7, 7, OutT, 7>(a, blocks, ldsBytes, in, w, bias, out, stream);
  if (a.d.kH == 7 && a.d.kW == 7 && unit && a.d.stripPixels == 4)
    return run<7, 7, OutT, 4>(a, blocks, ldsBytes, in, w, bias, out, stream);
  if (a.d.kH == 5 && a.d.kW == 5)
    return run<5, 5, OutT>(a, blocks, ldsBytes, in, w, bias, out, stream);
  return run<0, 0, OutT>(a, blocks, ldsBytes, in, w, bias, out, stream);
}

} // namespace

bool depthwiseStripTakes(const DepthwiseDesc &d) {
  return d.kH == 7 && d.kW == 7 && d.strideH == 1 && d.strideW == 1 &&
         d.dilH == 1 && d.dilW == 1 && d.inDilH == 1 && d.inDilW == 1 &&
         d.channels % 8 == 0 && d.elemBytes == 2;
}

uint64_t depthwiseTileLdsBytes(const DepthwiseDesc &d) {
  const uint64_t vecs = uint64_t(d.channels) * d.elemBytes / 16,
                 vecBlock = vecs <= 16 ? vecs : 16;
  const uint64_t patchH = uint64_t(d.tileH - 1) * d.strideH +
                          uint64_t(d.kH - 1) * d.dilH + 1;
  const uint64_t patchW = uint64_t(d.tileW - 1) * d.strideW +
                          uint64_t(d.kW - 1) * d.dilW + 1;
  const uint64_t rowPitch = (patchW * vecBlock + 63) / 64 * 64;
  return patchH * rowPitch * 16 +
         (d.stripPixels ? uint64_t(d.kH) * d.kW * vecBlock * 16 : 0);
}

hipError_t launchDepthwise(const DepthwiseDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, const QuarterInfo &q,
                           hipStream_t stream) {
  // The kernels address a launch's tensors with 32-bit offsets.  Images are
  // independent: a batch whose input or output exceeds that goes out as
  // several launches of as many images as fit.
  {
    const uint64_t outBytes = outType == kHalf ? 2 : 4;
    const uint64_t inImage = uint64_t(d.inH) * d.inW * d.channels * d.elemBytes;
    const uint64_t outImage = uint64_t(d.outH) * d.outW * d.channels * outBytes;
    const uint64_t limit = kOutOfRange / 2;
    const uint64_t image = inImage > outImage ? inImage : outImage;
    if (image != 0 && image < limit && uint64_t(d.batch) * image >= limit) {
      const uint32_t perLaunch = uint32_t(limit / image);
      for (uint32_t first = 0; first < d.batch; first += perLaunch) {
        DepthwiseDesc part = d;
        part.batch = d.batch - first < perLaunch ? d.batch - first : perLaunch;
        const hipError_t e = launchDepthwise(
            part, inType, outType,
            static_cast<const char *>(in) + first * inImage, weightsPacked,
            bias, static_cast<char *>(out) + first * outImage, q, stream);
        if (e != hipSuccess)
          return e;
      }
      return hipSuccess;
    }
  }
  if (d.inDilH != 1 || d.inDilW != 1)
    return launchDepthwiseDirect(d, inType, outType, in, weightsPacked, bias,
                                 out, stream);
  if (d.dense3x3 == 2)
    return launchDepthwiseRows(d, inType, outType, in, weightsPacked, bias,
                               out, stream);
  if (d.dense3x3)
    return launchDepthwise3x3(d, inType, outType, in, weightsPacked, bias,
                                 out, stream);
  const uint32_t elemBytes = inType == kHalf ? 2 : inType == kFloat ? 4 : 1;
  const uint32_t perVec = 16 / elemBytes;
  if (d.elemBytes != elemBytes || d.channels % perVec != 0 || d.tileH == 0 ||
      d.tileW == 0 || (inType == kQuarter && outType != kHalf))
    return hipErrorInvalidValue;
  if (uint64_t(d.batch) * d.outH * d.outW * d.channels == 0)
    return hipSuccess;
  DwArgs a;
  a.d = d;
  a.formatIn = q.inFormat == kE4M3 ? 1 : 0;
  a.formatWeights = q.weightFormat == kE4M3 ? 1 : 0;
  a.scale = inType == kQuarter ? q.scale : 1.0f;
  a.vecs = d.channels / perVec;
  a.vecBlock = a.vecs <= 16 ? a.vecs : 16;
  a.vecShift = 4;
  a.vecBlocks = (a.vecs + a.vecBlock - 1) / a.vecBlock;
  a.tilesH = (d.outH + d.tileH - 1) / d.tileH;
  a.tilesW = (d.outW + d.tileW - 1) / d.tileW;
  a.patchH = (d.tileH - 1) * d.strideH + (d.kH - 1) * d.dilH + 1;
  a.patchW = (d.tileW - 1) * d.strideW + (d.kW - 1) * d.dilW + 1;
  a.rowElems = a.patchW * a.vecBlock;
  a.rowPitch = (a.rowElems + 63) / 64 * 64;
  a.pixelsPerRound = kThreads / a.vecBlock;
  a.stepY = a.pixelsPerRound / d.tileW;
  a.stepX = a.pixelsPerRound % d.tileW;
  const uint64_t inBytes =
      uint64_t(d.batch) * d.inH * d.inW * d.channels * elemBytes;
  const uint64_t ldsBytes = uint64_t(a.patchH) * a.rowPitch * 16;
  const uint64_t blocks =
      uint64_t(d.batch) * a.tilesH * a.tilesW * a.vecBlocks;
  if (inBytes >= kOutOfRange || blocks > 0x7fffffffull ||
      depthwiseTileLdsBytes(d) > (d.stripPixels ? kLdsMost : 64 * 1024) ||
      (d.stripPixels != 0 && !depthwiseStripTakes(d)))
    return hipErrorInvalidConfiguration;
  a.inBytes = uint32_t(inBytes);
  if (inType == kFloat && outType == kFloat)
    return runOtherType<float, float>(a, uint32_t(blocks), uint32_t(ldsBytes),
                                      in, weightsPacked, bias, out, stream);
  if (inType == kFloat && outType == kHalf)
    return runOtherType<__half, float>(a, uint32_t(blocks), uint32_t(ldsBytes),
                                       in, weightsPacked, bias, out, stream);
  if (inType == kQuarter)
    return runOtherType<__half, uint8_t>(a, uint32_t(blocks),
                                         uint32_t(ldsBytes), in, weightsPacked,
                                         bias, out, stream);
  if (outType == kHalf)
    return runKernelShape<__half>(a, uint32_t(blocks), uint32_t(ldsBytes), in,
                                  weightsPacked, bias, out, stream);
  if (outType == kFloat)
    return runKernelShape<float>(a, uint32_t(blocks), uint32_t(ldsBytes), in,
                                 weightsPacked, bias, out, stream);
  return hipErrorInvalidValue;
}

} // namespace mxk

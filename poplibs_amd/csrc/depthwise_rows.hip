// Depthwise 3x3 forward convolution (dilation 1, stride 1 or 2) by persistent
// workgroups that stream input rows through a ring in LDS: the same role as
// depthwise3x3.hip (PopLibs' HorizontalMac vertices,
// lib/poplin/codelets/ConvPartialHorizontalMac.cpp:34-133), for layers large
// enough to give every CU a band of rows.
//
// A workgroup owns a band of output rows of one column strip of one image
// and walks down it.  Loader waves bring the strip's input rows, one after
// the other, into a ring of row slots with dense 1 KB loads that write LDS
// directly (no registers, so many rows are in flight); every input row is
// fetched once per band - the two (stride 2) or one (stride 1) new rows an
// output row needs, not the three it reads.  Compute waves - one thread per
// output pixel and channel vector of the current output row - read their nine
// input vectors from the ring, multiply by taps they keep in registers for
// the whole band, and store 16 bytes each, a whole output row of the strip as
// one contiguous run.  One barrier per output row.  Several loader waves,
// because one wave does not issue loads as fast as HBM delivers them (ten
// instructions per load).
//
// depthwiseRowsDeltaKernel is the same walk for the layer's weight deltas,
//   dW[kh][kw][c] = sum over b, oh, ow of
//       deltas[b][oh][ow][c] * acts[b][oh S + kh - padH][ow S + kw - padW][c]
// (the pass PopLibs runs as a convolution of its own,
// lib/poplin/Convolution.cpp:3437-3483 calculateWeightDeltas): a second,
// smaller ring holds the rows of the deltas, a thread keeps the 9 x 8 sums of
// its output column and channel vector in registers down the band, the
// columns meet in LDS at the end, and every workgroup leaves one [9][C] fp32
// tile, which depthwiseDeltaSumKernel adds in order.
#include "igemm_common.hpp"

namespace mxk {
namespace {

constexpr int kRowLoads = 12;           // 1 KB loads per input row slot
constexpr int kSlotBytes = kRowLoads * 1024;
constexpr int kLoaderWaves = 4;
constexpr int kComputeWaves = 6;
constexpr int kComputeThreads = 64 * kComputeWaves;
constexpr int kRowsThreads = 64 * (kComputeWaves + kLoaderWaves);
constexpr int kOwnLoads = kRowLoads / kLoaderWaves; // per loader wave and row
constexpr uint32_t kNoByte = 0x80000000u;           // beyond any buffer here

// Wall-clock stamps (s_memrealtime, 100 MHz) of depthwiseRowsKernel's
// milestones, for the build with -DMXK_ROWS_STAMPS only
// (libmxconv_stamps.so; the product library carries none of this): compute
// wave 0 and the first loader wave of every workgroup write eight stamps each
// to the buffer mxk_rows_stamp_sink() names: [workgroup][compute | loader][8].
#ifdef MXK_ROWS_STAMPS
__device__ uint64_t *rowsStampSink = nullptr;
#define MXK_RSTAMP_DECL uint64_t rstamps_[8] = {}
#define MXK_RSTAMP(i) rstamps_[i] = __builtin_amdgcn_s_memrealtime()
#define MXK_RSTAMP_IF(c, i)                                                    \
  if (c)                                                                       \
  rstamps_[i] = __builtin_amdgcn_s_memrealtime()
#define MXK_RSTAMP_OUT(who, on)                                                \
  if (rowsStampSink && (on))                                                   \
    for (int i_ = 0; i_ != 8; ++i_)                                            \
  rowsStampSink[(size_t(blockIdx.x) * 2 + (who)) * 8 + i_] = rstamps_[i_]
#else
#define MXK_RSTAMP_DECL
#define MXK_RSTAMP(i)
#define MXK_RSTAMP_IF(c, i)
#define MXK_RSTAMP_OUT(who, on)
#endif

/// The forward kernel's ring by stride.  kAhead: steps (output rows) the
/// loads run ahead; a step needs rows [j S, j S + 2], so `ahead` steps on the
/// way take ahead * S + 3 slots.  Six rows on the way: on N = 32, 112 x 112,
/// 96 channels, stride 2 that takes 17.7 us, eight rows 18.0, ten 18.3, four
/// 17.85, two 18.9; two loader waves 18.2, six as four.
/// At stride 1 a step adds one row to the two the step before it used: the
/// compute waves keep the window in registers and read the row the NEXT step
/// adds while they multiply (kEarlyRows = 1: that row has landed a step
/// early, one more slot), and eight compute waves, two on every SIMD, take
/// wider strips (N = 32, 56 x 56, 144 channels: 16.5 us with six waves
/// reading nine vectors per step, 13.8 with eight, 13.1 with the register
/// window as well).  At stride 2 both cost time (17.8 -> 18.0 and 18.2 us).
/// (Strips of channels as well as of columns, so that wide pixels get wider
/// column strips and fewer halo columns, lose: pieces of 256 to 640 bytes of
/// every pixel read by different workgroups - N = 32, 28 x 28, 512 channels
/// 11.5 -> 12.7 us, N = 128, 14 x 14, 576 channels 12.2 -> 16.8 us.)
/// (K: the kernel is K x K, 3 or 5.  At 5 x 5 the 25 taps fill the registers
/// the window would want, so both strides read their window from LDS; eight
/// compute waves at stride 1 as for 3 x 3.)
template <int S, int K = 3> struct Ring {
  static constexpr int kAhead = 6 / S;
  static constexpr int kEarlyRows = S == 1 && K == 3 ? 1 : 0;
  static constexpr int kWindow = K + kEarlyRows; // rows landed at a barrier
  static constexpr int kSlots = kAhead * S + kWindow;
  static constexpr int kComputeWaves = S == 1 ? 8 : 6;
  static constexpr int kComputeThreads = 64 * kComputeWaves;
  static constexpr int kThreads = 64 * (kComputeWaves + kLoaderWaves);
  static_assert(kSlots * kSlotBytes <= 160 * 1024, "LDS of a CU");
};
constexpr uint32_t fwdComputeThreads(uint32_t stride) {
  return stride == 1 ? Ring<1>::kComputeThreads : Ring<2>::kComputeThreads;
}

struct RowsArgs {
  DepthwiseDesc d;
  uint32_t vecs;              // channels / 8
  uint32_t strips, colsOut;   // column strips per image, output columns each
  uint32_t bands, rowsOut;    // row bands per strip, output rows each
  uint32_t colsIn;            // input columns of a strip: (colsOut-1)*S + 3
  uint32_t inBytes;
  FastDiv divVecs, divStrips, divBands;
};

union Vec8 {
  uintx4 raw;
  __half2 h2[4];
};

template <class OutT> struct PutVec;
template <> struct PutVec<__half> {
  static __device__ __forceinline__ void put(__half *p, const float (&v)[8]) {
    Vec8 o;
#pragma unroll
    for (int i = 0; i != 4; ++i)
      o.h2[i] = roundPairToHalf(v[2 * i], v[2 * i + 1]);
    __builtin_nontemporal_store(o.raw, reinterpret_cast<uintx4 *>(p));
  }
};
template <> struct PutVec<float> {
  static __device__ __forceinline__ void put(float *p, const float (&v)[8]) {
    __builtin_nontemporal_store(floatx4{v[0], v[1], v[2], v[3]},
                                reinterpret_cast<floatx4 *>(p));
    __builtin_nontemporal_store(floatx4{v[4], v[5], v[6], v[7]},
                                reinterpret_cast<floatx4 *>(p + 4));
  }
};

/// What a loader wave knows of a strip's rows of one tensor: per own load,
/// the byte of its 16-byte unit from the row's first pixel, or kNoByte.
/// LOADS: loads per row and loader wave; row slots are LOADS * kLoaderWaves KB.
template <int LOADS> struct StripRow {
  uint32_t unitByte[LOADS];
  /// Columns [first, first + cols) of rows whose valid columns are [lo, hi).
  __device__ __forceinline__ void setup(int first, uint32_t cols, int lo,
                                        int hi, uint32_t pixelBytes,
                                        uint32_t vecs, const FastDiv &divVecs,
                                        int loader, uint32_t lane) {
#pragma unroll
    for (int own = 0; own != LOADS; ++own) {
      const uint32_t u = (own * kLoaderWaves + loader) * 64 + lane;
      const uint32_t col = divVecs(u);
      const int at = first + int(col);
      unitByte[own] = col < cols && at >= lo && at < hi
                          ? uint32_t(at) * pixelBytes + (u - col * vecs) * 16
                          : kNoByte;
    }
  }
  /// The row that starts at rowByte of the buffer (kNoByte: a row of zeros)
  /// into `slot`.
  __device__ __forceinline__ void load(const __amdgpu_buffer_rsrc_t &buf,
                                       char *slot, uint32_t rowByte,
                                       int loader) const {
#pragma unroll
    for (int own = 0; own != LOADS; ++own)
      // (anything with kNoByte in it lies beyond the buffer: zeros)
      loadToLds<kStreamingLoad>(
          buf, (LdsPtr)(slot + (own * kLoaderWaves + loader) * 1024),
          (rowByte | unitByte[own]) >= kNoByte ? kNoByte
                                               : rowByte + unitByte[own],
          0);
  }
};

template <int S, int K, class OutT>
__global__ __launch_bounds__((Ring<S, K>::kThreads)) void depthwiseRowsKernel(
    RowsArgs a, const __half *__restrict__ in, const __half *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out) {
  using R = Ring<S, K>;
  constexpr int kAhead = R::kAhead, kSlots = R::kSlots;
  extern __shared__ __align__(16) char lds[];
  const DepthwiseDesc &d = a.d;
  const uint32_t t = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(int(t >> 6));
  const uint32_t lane = t & 63;

  // Workgroup -> (image, band, strip), strip fastest; each XCD, which takes
  // workgroups round-robin, gets a contiguous run: neighbouring bands share
  // their halo rows in its L2.
  const uint32_t walker = xcdSwizzle(blockIdx.x, gridDim.x);
  uint32_t q = a.divStrips(walker);
  const uint32_t strip = walker - q * a.strips;
  const uint32_t b = a.divBands(q);
  const uint32_t band = q - b * a.bands;
  const uint32_t oh0 = band * a.rowsOut, ow0 = strip * a.colsOut;
  const uint32_t steps =
      oh0 + a.rowsOut <= d.outH ? a.rowsOut : d.outH - oh0;
  const int ih0 = int(oh0 * S) - d.padH, iw0 = int(ow0 * S) - d.padW;
  const uint32_t pixelBytes = d.channels * 2;
  // relative input rows [0, rowsIn) are what the band reads
  const uint32_t rowsIn = (steps - 1) * S + K;

  MXK_RSTAMP_DECL;
  MXK_RSTAMP(0); // the wave starts
  if (wave >= R::kComputeWaves) {
    // ---- loaders.  Load L of a row fills bytes [1024 L, 1024 L + 1024) of
    // its slot: 16-byte unit u = 64 L + lane is channel vector u % vecs of
    // strip column u / vecs.  Loader l takes L = l, l + kLoaderWaves, ...
    const int loader = wave - R::kComputeWaves;
    const __amdgpu_buffer_rsrc_t inBuf = bufferOf(in, a.inBytes);
    StripRow<kOwnLoads> strip;
    strip.setup(iw0, a.colsIn, int(d.loW), int(d.hiW), pixelBytes, a.vecs,
                a.divVecs, loader, lane);
    const uint32_t imageByte = b * d.inH * d.inW * pixelBytes;
    const uint32_t rowBytes = d.inW * pixelBytes;
    MXK_RSTAMP(1); // set-up done: the first load goes out
    uint32_t next = 0; // the relative row loaded next
    auto loadRow = [&] {
      const int ih = ih0 + int(next);
      const bool ok = next < rowsIn && ih >= int(d.loH) && ih < int(d.hiH);
      const uint32_t rowByte =
          ok ? imageByte + uint32_t(ih) * rowBytes : kNoByte;
      strip.load(inBuf, lds + (next % kSlots) * kSlotBytes, rowByte, loader);
      ++next;
    };
    // rows of steps 0 .. kAhead - 1
#pragma unroll 1
    for (int r = 0; r != (kAhead - 1) * S + R::kWindow; ++r) {
      loadRow();
      MXK_RSTAMP_IF(r == R::kWindow - 1, 2); // step 0's rows requested
    }
    MXK_RSTAMP(3); // the rows of the first kAhead steps requested
    for (uint32_t j = 0; j < steps; ++j) {
      // step j's window has landed when all but the rows of the kAhead - 1
      // steps behind it have
      MXK_WAIT_VMCNT((kAhead - 1) * S * kOwnLoads);
      stepBarrier();
      // (the rows before step j's are free: everybody is through step j - 1)
#pragma unroll
      for (int r = 0; r != S; ++r)
        loadRow();
    }
    MXK_RSTAMP(4); // last loads issued
    MXK_WAIT_VMCNT(0);
    MXK_RSTAMP(5); // ... and landed
    MXK_RSTAMP_OUT(1, wave == R::kComputeWaves && lane == 0);
    return;
  }

  // ---- compute waves.  Thread t: strip column t / vecs, channel vector
  // t % vecs.
  const uint32_t col = a.divVecs(t), v = t - col * a.vecs;
  const uint32_t ow = ow0 + col;
  const bool active = col < a.colsOut && ow < d.outW;
  const uint32_t c = (active ? v : 0) * 8;
  Vec8 taps[K * K];
#pragma unroll
  for (int tap = 0; tap != K * K; ++tap)
    taps[tap].raw =
        *reinterpret_cast<const uintx4 *>(w + tap * d.channels + c);
  float biasV[8];
#pragma unroll
  for (int e = 0; e != 8; ++e)
    biasV[e] = bias ? Load<OutT>::at(bias, c + e, 0) : 0.0f;
  // the thread's window in a row slot: columns col * S .. + 2
  const uint32_t windowByte = ((active ? col : 0) * S * a.vecs + v) * 16;
  OutT *dst = out + ((size_t(b) * d.outH + oh0) * d.outW + ow) * d.channels + c;
  const size_t outRow = size_t(d.outW) * d.channels;
  auto rowOf = [&](uint32_t slot) {
    return lds + slot * kSlotBytes + windowByte;
  };
  auto readRow = [&](Vec8(&row)[K], const char *from) {
#pragma unroll
    for (int kw = 0; kw != K; ++kw)
      row[kw].raw =
          *reinterpret_cast<const uintx4 *>(from + kw * a.vecs * 16);
  };
  // out row = bias + the taps over the window's rows, kh then kw; row kh of
  // the window is rows[(first + kh) % ROWS]
  auto multiply = [&](auto &rows, auto firstRow) {
    constexpr int FIRST = decltype(firstRow)::value;
    constexpr int ROWS = int(sizeof(rows) / sizeof(rows[0]));
    float acc[8];
#pragma unroll
    for (int e = 0; e != 8; ++e)
      acc[e] = biasV[e];
#pragma unroll
    for (int kh = 0; kh != K; ++kh)
#pragma unroll
      for (int kw = 0; kw != K; ++kw) {
        const Vec8 &x = rows[(FIRST + kh) % ROWS][kw];
        const Vec8 &k = taps[kh * K + kw];
#pragma unroll
        for (int e = 0; e != 4; ++e) {
          const float2 xf = __half22float2(x.h2[e]);
          const float2 kf = __half22float2(k.h2[e]);
          acc[2 * e] = fmaf(xf.x, kf.x, acc[2 * e]);
          acc[2 * e + 1] = fmaf(xf.y, kf.y, acc[2 * e + 1]);
        }
      }
    if (active)
      PutVec<OutT>::put(dst, acc);
    dst += outRow;
  };
  auto next = [&](uint32_t slot) {
    return slot + 1 == uint32_t(kSlots) ? 0u : slot + 1;
  };

  if constexpr (R::kEarlyRows == 0) {
    // A step reads its K rows behind its barrier.  (The reads are done -
    // their values were used - before the next barrier lets the loaders
    // overwrite the rows.)
    uint32_t slot = 0; // slot of relative row j * S
    for (uint32_t j = 0; j < steps; ++j) {
      stepBarrier(); // step j's rows are in the ring
      MXK_RSTAMP_IF(j == 0, 1);         // step 0's rows have landed
      MXK_RSTAMP_IF(j == 1, 2);         // step 1's
      MXK_RSTAMP_IF(j + 1 == steps, 3); // the last step's
      uint32_t rowSlot = slot;
      if constexpr (K == 3) {
        Vec8 win[K][K];
#pragma unroll
        for (int kh = 0; kh != K; ++kh) {
          readRow(win[kh], rowOf(rowSlot));
          rowSlot = next(rowSlot);
        }
        multiply(win, std::integral_constant<int, 0>{});
      } else {
        // (the 25 taps leave no room for the whole window, nor for a second
        // row to read ahead: a row at a time, the other waves' work under
        // the reads)
        // (the taps stay packed halves: as loop constants the compiler
        // would keep fp32 copies of them, 200 registers)
#pragma unroll
        for (int tap = 0; tap != K * K; ++tap)
          asm volatile("" : "+v"(taps[tap].raw));
        float acc[8];
#pragma unroll
        for (int e = 0; e != 8; ++e)
          acc[e] = biasV[e];
#pragma unroll
        for (int kh = 0; kh != K; ++kh) {
          Vec8 row[K];
          readRow(row, rowOf(rowSlot));
          rowSlot = next(rowSlot);
#pragma unroll
          for (int kw = 0; kw != K; ++kw) {
            const Vec8 &x = row[kw];
            const Vec8 &k = taps[kh * K + kw];
#pragma unroll
            for (int e = 0; e != 4; ++e) {
              const float2 xf = __half22float2(x.h2[e]);
              const float2 kf = __half22float2(k.h2[e]);
              acc[2 * e] = fmaf(xf.x, kf.x, acc[2 * e]);
              acc[2 * e + 1] = fmaf(xf.y, kf.y, acc[2 * e + 1]);
            }
          }
        }
        if (active)
          PutVec<OutT>::put(dst, acc);
        dst += outRow;
      }
      slot += S;
      slot -= slot >= uint32_t(kSlots) ? kSlots : 0;
    }
  } else {
    // Stride 1.  The window lives in four register rows: a step multiplies
    // the three it holds from earlier steps and reads the one the next step
    // adds into the fourth, so every row is read from LDS once and that read
    // hides behind the multiplications.  A row's slot is loaded into again
    // only after the barrier of the step behind the one that used the row.
    static_assert(S == 1 && K == 3 && R::kEarlyRows == 1, "one row per step");
    Vec8 win[4][3];
    uint32_t readSlot = 0; // slot of the next row to read
    auto step = [&](auto off, bool first) {
      constexpr int OFF = decltype(off)::value;
      stepBarrier(); // the step's rows and the next step's are in the ring
      if (first) {
#pragma unroll
        for (int r = 0; r != 3; ++r) {
          readRow(win[r], rowOf(readSlot));
          readSlot = next(readSlot);
        }
      }
      readRow(win[(OFF + 3) % 4], rowOf(readSlot));
      readSlot = next(readSlot);
      multiply(win, off);
    };
    // the register rows come round every four steps
    for (uint32_t j = 0; j < steps; j += 4) {
      step(std::integral_constant<int, 0>{}, j == 0);
      if (j + 1 < steps)
        step(std::integral_constant<int, 1>{}, false);
      if (j + 2 < steps)
        step(std::integral_constant<int, 2>{}, false);
      if (j + 3 < steps)
        step(std::integral_constant<int, 3>{}, false);
    }
  }
#ifdef MXK_ROWS_STAMPS
  MXK_RSTAMP(4); // last store issued
  __builtin_amdgcn_s_waitcnt(0);
  MXK_RSTAMP(5); // ... and landed
  MXK_RSTAMP_OUT(0, t == 0);
#endif
}


// ---- weight deltas

constexpr int kDeltaLoads = 8; // 1 KB loads per slot of a row of deltas
constexpr int kDeltaSlotBytes = kDeltaLoads * 1024;
constexpr int kOwnDeltaLoads = kDeltaLoads / kLoaderWaves;
constexpr int kSumRow = 73; // floats a thread leaves for the columns' meeting

/// Rings of the weight-delta kernel: rows of activations as in the forward
/// kernel, one row of deltas per step; four steps' rows on the way at stride
/// 1, three at stride 2 (124 / 140 KB of LDS).  Eight compute waves at stride
/// 1, as in the forward kernel (a step moves half a stride-2 step's bytes for
/// the same multiply-adds); the rings' memory is where the columns' sums meet
/// at the end, 73 floats per compute thread.
template <int S> struct DeltaRing {
  static constexpr int kAhead = S == 2 ? 3 : 4;
  static constexpr int kSlots = kAhead * S + 3;
  static constexpr int kDeltaSlots = kAhead + 1;
  static constexpr int kComputeWaves = S == 1 ? 8 : 6;
  static constexpr int kComputeThreads = 64 * kComputeWaves;
  static constexpr int kThreads = 64 * (kComputeWaves + kLoaderWaves);
  static constexpr int kRingBytes =
      kSlots * kSlotBytes + kDeltaSlots * kDeltaSlotBytes;
  static constexpr int kSumBytes = kComputeThreads * kSumRow * 4;
  static constexpr int kBytes = kRingBytes > kSumBytes ? kRingBytes : kSumBytes;
  static_assert(kComputeThreads * 16 <= kDeltaSlotBytes,
                "every compute thread has a unit of a row of deltas");
  static_assert(kBytes <= 160 * 1024, "LDS of a CU");
};
constexpr uint32_t deltaComputeThreads(uint32_t stride) {
  return stride == 1 ? DeltaRing<1>::kComputeThreads
                     : DeltaRing<2>::kComputeThreads;
}

/// partial[walker][tap][c] = the walker's band's sum.
template <int S>
__global__ __launch_bounds__(DeltaRing<S>::kThreads) void depthwiseRowsDeltaKernel(
    RowsArgs a, const __half *__restrict__ acts,
    const __half *__restrict__ deltas, uint32_t deltaBytes,
    float *__restrict__ partial) {
  using R = DeltaRing<S>;
  constexpr int kAhead = R::kAhead, kSlots = R::kSlots;
  constexpr int kDeltaSlots = R::kDeltaSlots;
  extern __shared__ __align__(16) char lds[];
  char *deltaRing = lds + kSlots * kSlotBytes;
  const DepthwiseDesc &d = a.d;
  const uint32_t t = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(int(t >> 6));
  const uint32_t lane = t & 63;

  const uint32_t walker = xcdSwizzle(blockIdx.x, gridDim.x);
  uint32_t q = a.divStrips(walker);
  const uint32_t strip = walker - q * a.strips;
  const uint32_t b = a.divBands(q);
  const uint32_t band = q - b * a.bands;
  const uint32_t oh0 = band * a.rowsOut, ow0 = strip * a.colsOut;
  const uint32_t steps =
      oh0 + a.rowsOut <= d.outH ? a.rowsOut : d.outH - oh0;
  const int ih0 = int(oh0 * S) - d.padH, iw0 = int(ow0 * S) - d.padW;
  const uint32_t pixelBytes = d.channels * 2;
  const uint32_t rowsIn = (steps - 1) * S + 3;

  if (wave >= R::kComputeWaves) {
    // ---- loaders: per step the new rows of activations, then the step's
    // row of deltas (output columns [ow0, ow0 + colsOut) of row oh0 + j).
    const int loader = wave - R::kComputeWaves;
    const __amdgpu_buffer_rsrc_t actBuf = bufferOf(acts, a.inBytes);
    const __amdgpu_buffer_rsrc_t deltaBuf = bufferOf(deltas, deltaBytes);
    StripRow<kOwnLoads> actStrip;
    actStrip.setup(iw0, a.colsIn, int(d.loW), int(d.hiW), pixelBytes, a.vecs,
                   a.divVecs, loader, lane);
    StripRow<kOwnDeltaLoads> deltaStrip;
    deltaStrip.setup(int(ow0), a.colsOut, 0, int(d.outW), pixelBytes, a.vecs,
                     a.divVecs, loader, lane);
    const uint32_t imageByte = b * d.inH * d.inW * pixelBytes;
    const uint32_t rowBytes = d.inW * pixelBytes;
    const uint32_t deltaImageByte = b * d.outH * d.outW * pixelBytes;
    const uint32_t deltaRowBytes = d.outW * pixelBytes;
    uint32_t next = 0, nextStep = 0;
    auto loadStep = [&](int rows) {
      for (int r = 0; r != rows; ++r) {
        const int ih = ih0 + int(next);
        const bool ok = next < rowsIn && ih >= int(d.loH) && ih < int(d.hiH);
        actStrip.load(actBuf, lds + (next % kSlots) * kSlotBytes,
                      ok ? imageByte + uint32_t(ih) * rowBytes : kNoByte,
                      loader);
        ++next;
      }
      deltaStrip.load(deltaBuf,
                      deltaRing + (nextStep % kDeltaSlots) * kDeltaSlotBytes,
                      nextStep < steps ? deltaImageByte +
                                             (oh0 + nextStep) * deltaRowBytes
                                       : kNoByte,
                      loader);
      ++nextStep;
    };
    // steps 0 .. kAhead - 1, in the order the loop goes on in: the counts
    // below rely on it
    loadStep(3);
#pragma unroll 1
    for (int s = 1; s != kAhead; ++s)
      loadStep(S);
    for (uint32_t j = 0; j < steps; ++j) {
      MXK_WAIT_VMCNT((kAhead - 1) * (S * kOwnLoads + kOwnDeltaLoads));
      stepBarrier();
      loadStep(S);
    }
    MXK_WAIT_VMCNT(0);
    // (the rings are the columns' meeting place next: nothing of these
    // loads' may land later)
    stepBarrier();
    return;
  }

  // ---- compute waves.  Thread t: strip column t / vecs, channel vector
  // t % vecs; a thread beyond the strip's columns reads zeros for deltas.
  const uint32_t colOf = a.divVecs(t), v = t - colOf * a.vecs;
  const bool inStrip = colOf < a.colsOut;
  const uint32_t col = inStrip ? colOf : 0;
  const uint32_t windowByte = (col * S * a.vecs + v) * 16;
  // (8 KB hold 512 units: any t has a unit, of zeros beyond the strip)
  const uint32_t deltaByte = t * 16;
  float acc[9][8];
#pragma unroll
  for (int tap = 0; tap != 9; ++tap)
#pragma unroll
    for (int e = 0; e != 8; ++e)
      acc[tap][e] = 0.0f;
  uint32_t slot = 0, deltaSlot = 0;
  for (uint32_t j = 0; j < steps; ++j) {
    stepBarrier();
    Vec8 dz;
    dz.raw = *reinterpret_cast<const uintx4 *>(
        deltaRing + deltaSlot * kDeltaSlotBytes + deltaByte);
    float dzf[8];
#pragma unroll
    for (int e = 0; e != 4; ++e) {
      const float2 f = __half22float2(dz.h2[e]);
      dzf[2 * e] = f.x, dzf[2 * e + 1] = f.y;
    }
    uint32_t rowSlot = slot;
#pragma unroll
    for (int kh = 0; kh != 3; ++kh) {
      const char *row = lds + rowSlot * kSlotBytes + windowByte;
#pragma unroll
      for (int kw = 0; kw != 3; ++kw) {
        Vec8 x;
        x.raw = *reinterpret_cast<const uintx4 *>(row + kw * a.vecs * 16);
#pragma unroll
        for (int e = 0; e != 4; ++e) {
          const float2 xf = __half22float2(x.h2[e]);
          acc[kh * 3 + kw][2 * e] =
              fmaf(xf.x, dzf[2 * e], acc[kh * 3 + kw][2 * e]);
          acc[kh * 3 + kw][2 * e + 1] =
              fmaf(xf.y, dzf[2 * e + 1], acc[kh * 3 + kw][2 * e + 1]);
        }
      }
      rowSlot = rowSlot + 1 == kSlots ? 0 : rowSlot + 1;
    }
    slot += S;
    slot -= slot >= kSlots ? kSlots : 0;
    deltaSlot = deltaSlot + 1 == kDeltaSlots ? 0 : deltaSlot + 1;
  }
  // The columns meet: every thread leaves its 72 sums, then thread o adds
  // those of output o = (tap, channel) over the strip's columns, in order.
  stepBarrier(); // the loaders' last (zero) rows have landed, all reads done
  float *sums = reinterpret_cast<float *>(lds);
#pragma unroll
  for (int tap = 0; tap != 9; ++tap)
#pragma unroll
    for (int e = 0; e != 8; ++e)
      sums[t * kSumRow + tap * 8 + e] = inStrip ? acc[tap][e] : 0.0f;
  __syncthreads();
  const uint32_t outputs = 9 * d.channels;
  float *dst = partial + size_t(walker) * outputs;
  for (uint32_t o = t; o < outputs; o += R::kComputeThreads) {
    const uint32_t tap = o / d.channels, c = o - tap * d.channels;
    const float *from = sums + (c >> 3) * kSumRow + tap * 8 + (c & 7);
    float sum = 0.0f;
    for (uint32_t k = 0; k != a.colsOut; ++k)
      sum += from[k * a.vecs * kSumRow];
    dst[o] = sum;
  }
}

/// Strips, bands and their sizes for a chip of `cus` compute units; false
/// when the kernel does not take the layer.
bool shapeFor(const DepthwiseDesc &d, uint32_t cus, RowsArgs &a,
              uint32_t computeThreads = kComputeThreads) {
  if ((d.kH != 3 && d.kH != 5) || d.kW != d.kH || d.dilH != 1 || d.dilW != 1 ||
      d.strideH != d.strideW || (d.strideH != 1 && d.strideH != 2) ||
      d.channels % 8 != 0 || d.channels == 0 || d.inDilH != 1 ||
      d.inDilW != 1 || d.batch == 0 || d.outH == 0 || d.outW == 0)
    return false;
  const uint32_t s = d.strideH;
  a.vecs = d.channels / 8;
  // a strip's input row fits a slot, its output row the compute threads
  const uint32_t unitsPerSlot = kSlotBytes / 16;
  if (a.vecs * d.kW > unitsPerSlot || a.vecs > computeThreads)
    return false;
  const uint32_t maxColsIn = unitsPerSlot / a.vecs;
  uint32_t maxColsOut = (maxColsIn - d.kW) / s + 1;
  if (maxColsOut > computeThreads / a.vecs)
    maxColsOut = computeThreads / a.vecs;
  a.strips = (d.outW + maxColsOut - 1) / maxColsOut;
  a.colsOut = (d.outW + a.strips - 1) / a.strips;
  a.colsIn = (a.colsOut - 1) * s + d.kW;
  // about one workgroup per CU
  const uint64_t columns = uint64_t(d.batch) * a.strips;
  uint64_t bands = cus / columns;
  if (bands < 1)
    bands = 1;
  if (bands > d.outH)
    bands = d.outH;
  a.rowsOut = uint32_t((d.outH + bands - 1) / bands);
  a.bands = (d.outH + a.rowsOut - 1) / a.rowsOut;
  return true;
}

template <int S, int K, class OutT>
hipError_t run(const RowsArgs &a, const void *in, const void *w,
               const void *bias, void *out, hipStream_t stream) {
  constexpr int ldsBytes = Ring<S, K>::kSlots * kSlotBytes;
  static const hipError_t attr = hipFuncSetAttribute(
      reinterpret_cast<const void *>(&depthwiseRowsKernel<S, K, OutT>),
      hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes);
  if (attr != hipSuccess)
    return attr;
  const uint32_t blocks = a.d.batch * a.strips * a.bands;
  hipLaunchKernelGGL((depthwiseRowsKernel<S, K, OutT>), dim3(blocks),
                     dim3(Ring<S, K>::kThreads), ldsBytes, stream, a,
                     static_cast<const __half *>(in),
                     static_cast<const __half *>(w),
                     static_cast<const OutT *>(bias), static_cast<OutT *>(out));
  return hipGetLastError();
}

} // namespace

namespace {
bool takes(const DepthwiseDesc &d, int inType, uint32_t computeThreads) {
  RowsArgs a;
  if (inType != kHalf || d.cus == 0 || !shapeFor(d, d.cus, a, computeThreads))
    return false;
  const uint64_t inBytes = uint64_t(d.batch) * d.inH * d.inW * d.channels * 2;
  const uint64_t blocks = uint64_t(d.batch) * a.strips * a.bands;
  return inBytes < kNoByte && blocks < 0x7fffffffull;
}

DepthwiseRowsLaunch launchShapeOf(const DepthwiseDesc &d,
                                  uint32_t computeThreads) {
  RowsArgs a{};
  DepthwiseRowsLaunch l{};
  if (d.cus == 0 || !shapeFor(d, d.cus, a, computeThreads))
    return l;
  l.strips = a.strips, l.colsOut = a.colsOut;
  l.bands = a.bands, l.rowsOut = a.rowsOut;
  l.workgroups = uint64_t(d.batch) * a.strips * a.bands;
  l.ringRows = d.kH == 5 ? (d.strideH == 2 ? Ring<2, 5>::kSlots : Ring<1, 5>::kSlots)
                         : (d.strideH == 2 ? Ring<2>::kSlots : Ring<1>::kSlots);
  l.loaderWaves = kLoaderWaves;
  l.computeWaves = computeThreads / 64;
  return l;
}
} // namespace

bool depthwiseRowsTakes(const DepthwiseDesc &d, int inType) {
  return takes(d, inType, fwdComputeThreads(d.strideH));
}

DepthwiseRowsLaunch depthwiseRowsLaunchShape(const DepthwiseDesc &d) {
  return launchShapeOf(d, fwdComputeThreads(d.strideH));
}

hipError_t launchDepthwiseRows(const DepthwiseDesc &d, int inType, int outType,
                               const void *in, const void *weightsPacked,
                               const void *bias, void *out,
                               hipStream_t stream) {
  if (!depthwiseRowsTakes(d, inType) ||
      (outType != kHalf && outType != kFloat))
    return hipErrorInvalidValue;
  RowsArgs a{};
  shapeFor(d, d.cus, a, fwdComputeThreads(d.strideH));
  a.d = d;
  a.inBytes = uint32_t(uint64_t(d.batch) * d.inH * d.inW * d.channels * 2);
  a.divVecs = makeFastDiv(a.vecs);
  a.divStrips = makeFastDiv(a.strips);
  a.divBands = makeFastDiv(a.bands);
  const bool s1 = d.strideH == 1, k3 = d.kH == 3;
  if (outType == kHalf)
    return s1 ? (k3 ? run<1, 3, __half>(a, in, weightsPacked, bias, out, stream)
                    : run<1, 5, __half>(a, in, weightsPacked, bias, out, stream))
              : (k3 ? run<2, 3, __half>(a, in, weightsPacked, bias, out, stream)
                    : run<2, 5, __half>(a, in, weightsPacked, bias, out,
                                        stream));
  return s1 ? (k3 ? run<1, 3, float>(a, in, weightsPacked, bias, out, stream)
                  : run<1, 5, float>(a, in, weightsPacked, bias, out, stream))
            : (k3 ? run<2, 3, float>(a, in, weightsPacked, bias, out, stream)
                  : run<2, 5, float>(a, in, weightsPacked, bias, out, stream));
}

bool depthwiseRowsDeltaTakes(const DepthwiseDesc &d) {
  const uint64_t deltaBytes =
      uint64_t(d.batch) * d.outH * d.outW * d.channels * 2;
  return d.kH == 3 && takes(d, kHalf, deltaComputeThreads(d.strideH)) &&
         deltaBytes < kNoByte;
}

DepthwiseRowsLaunch depthwiseRowsDeltaLaunchShape(const DepthwiseDesc &d) {
  DepthwiseRowsLaunch l = launchShapeOf(d, deltaComputeThreads(d.strideH));
  l.ringRows = d.strideH == 2 ? DeltaRing<2>::kSlots : DeltaRing<1>::kSlots;
  return l;
}

size_t depthwiseRowsDeltaWorkspaceBytes(const DepthwiseDesc &d) {
  const DepthwiseRowsLaunch l = depthwiseRowsDeltaLaunchShape(d);
  return size_t(l.workgroups) * 9 * d.channels * sizeof(float);
}

hipError_t launchDepthwiseRowsDeltas(const DepthwiseDesc &d, const void *acts,
                                     const void *deltas, void *partial,
                                     uint32_t *walkers, hipStream_t stream) {
  if (!depthwiseRowsDeltaTakes(d) || !partial)
    return hipErrorInvalidValue;
  RowsArgs a{};
  shapeFor(d, d.cus, a, deltaComputeThreads(d.strideH));
  a.d = d;
  a.inBytes = uint32_t(uint64_t(d.batch) * d.inH * d.inW * d.channels * 2);
  a.divVecs = makeFastDiv(a.vecs);
  a.divStrips = makeFastDiv(a.strips);
  a.divBands = makeFastDiv(a.bands);
  const uint32_t deltaBytes =
      uint32_t(uint64_t(d.batch) * d.outH * d.outW * d.channels * 2);
  const uint32_t blocks = d.batch * a.strips * a.bands;
  *walkers = blocks;
  auto run = [&](auto stride) -> hipError_t {
    constexpr int S = decltype(stride)::value;
    static const hipError_t attr = hipFuncSetAttribute(
        reinterpret_cast<const void *>(&depthwiseRowsDeltaKernel<S>),
        hipFuncAttributeMaxDynamicSharedMemorySize, DeltaRing<S>::kBytes);
    if (attr != hipSuccess)
      return attr;
    hipLaunchKernelGGL(depthwiseRowsDeltaKernel<S>, dim3(blocks),
                       dim3(DeltaRing<S>::kThreads), DeltaRing<S>::kBytes,
                       stream, a,
                       static_cast<const __half *>(acts),
                       static_cast<const __half *>(deltas), deltaBytes,
                       static_cast<float *>(partial));
    return hipGetLastError();
  };
  return d.strideH == 1 ? run(std::integral_constant<int, 1>{})
                        : run(std::integral_constant<int, 2>{});
}

} // namespace mxk

#ifdef MXK_ROWS_STAMPS
/// Stamps build only: the device buffer the stamped kernel writes to
/// ([workgroups][2][8] of 8 bytes), or null to switch the stamps off.
extern "C" int mxk_rows_stamp_sink(void *deviceBuffer) {
  return int(hipMemcpyToSymbol(HIP_SYMBOL(mxk::rowsStampSink), &deviceBuffer,
                               sizeof(deviceBuffer)));
}
#endif

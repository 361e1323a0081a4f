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
// MFMA lane wants them: 16 bytes = 8 halves (16 fp8, 4 floats) of
// consecutive k.  A field with a depth adds od / kd to pixels and taps in the
// same way.
//
// Workgroup: 512 threads = 8 wave64, tile 128 (M) x BN (N), BN = 64 or 128,
// K step of 128 bytes per row (64 halves / 128 fp8 / 32 floats).
//
// Producer / consumer waves.  Waves 4-7 only move data; waves 0-3 only feed
// the matrix cores (and run the epilogue); each SIMD holds one of each kind,
// so MFMAs and memory instructions overlap even when the problem offers no
// more than one workgroup per CU.  The two kinds meet at one workgroup
// barrier per k-step.
//
// Data path.  Every k-step the producers gather the im2col A tile and the B
// tile with 16-byte buffer loads that write straight into LDS
// (buffer_load_dwordx4 ... lds): no staging registers, so the depth of the
// prefetch is set by LDS capacity - all stages but one are in flight while
// one is being multiplied.  Such a load puts lane l's 16 bytes at LDS base +
// 16 l, i.e. one instruction fills 8 consecutive 128-byte tile rows.  LDS has
// 64 banks of 4 bytes (256 bytes per clock); an MFMA-operand read (32 rows,
// same k, 16 bytes per lane) runs at that rate only if each run of 16 lanes
// covers all 64 banks.  So the 16-byte chunks of row r are stored at position
// (chunk ^ (r & 7)), and in every second 8-row block rows 2i and 2i+1 swap
// places, which moves that block's chunks to the other 128 bytes of the
// 256-byte bank period.  The permutation is applied on the global side, by
// choosing which row and chunk each lane fetches, and undone in the LDS read
// address.
// Each consumer wave multiplies its 64 x BN/2 sub-tile with
// v_mfma_f32_32x32x16_f16 (fp16) or v_mfma_f32_32x32x64_f8f6f4 (fp8),
// accumulating in fp32.
//
// Addressing.  Everything per-row is computed once, before the loop, by one
// thread per row (the result is handed to the producers through a small LDS
// table): a byte offset and a bit mask "kernel tap t reads inside the input".  In the loop
// the wave-uniform part of the address (kernel tap, channel block) travels in
// the scalar offset of the buffer load, and a row whose tap falls on padding
// gets an out-of-range vector offset, for which the buffer unit delivers
// zeros - no branch and no select on data.  When a k-step spans several
// kernel taps (fewer than 128 bytes of channels per tap) the tap is per-lane
// and the offsets are formed in vector registers.
// Two more ways of addressing serve what the tap mask cannot.  A kernel of
// more than 32 taps (a weight update pass: its "kernel" is a whole output
// field) keeps, per row, the ranges of kernel rows and columns that read
// inside the input - a window is valid on an interval of each - and tests
// the tap against them.  A dilated (zero-stuffed) input (the backward pass of
// a strided layer) keeps each row's image offset and window origin, and the
// producers work out every tap's input position and validity arithmetically.
// A producer wave gets few issue slots next to a consumer's MFMAs, so both
// are written to need as few vector instructions per load as they can.
//
// Split K.  A convolution with few output tiles but a long K (a weight update
// pass, a skinny matrix product) is cut along K into `splitK` parts, one
// workgroup each; every part writes its fp32 partial tile to a workspace
// [part][pixel][channel] and a second kernel adds the parts in order.
//
// Epilogue.  The accumulators are scaled, biased, converted and written to
// LDS, then all 8 waves copy whole 16-byte vectors to the channels-last
// output, so that every store instruction covers full rows of the tile.
// Row m of the GEMM is output pixel m - or, for the caller that runs one
// convolution per phase of a zero-stuffed input or has a padded output field,
// every outStep-th pixel of a larger field from an offset; a weight update
// pass asks for the transposed result, [channel][pixel].
//
// This takes the role of PopLibs' AMP vertices ConvPartial1x1Out /
// ConvPartialnx1 (lib/poplin/codelets/ConvPartial1x1Out.cpp:49-173,
// ConvPartialnx1.cpp:52-246), including the quarter (fp8) case whose scale
// 2^(sIn + sW) is applied once to the fp32 sum
// (lib/poplin/codelets/inlineAssemblerConv.hpp:28-33).
#include "igemm_common.hpp"

namespace mxk {
namespace {

/// UNI: every k-step lies inside one kernel tap (Ci * EB is a multiple of
/// 128 bytes), so tap and channel block are wave-uniform.
/// The work of one workgroup: tile number `block` of the `blocks` tiles of
/// convolution `a`.
template <int BN, int NS, int EB, int FA, int FB, bool UNI, class OutT>
__device__ __forceinline__ void igemmTile(
    const IgemmArgs a, const char *__restrict__ in,
    const char *__restrict__ w, const OutT *__restrict__ bias,
    OutT *__restrict__ out, float scale, uint32_t block, uint32_t blocks) {
  constexpr int TN = BN / 64;              // 32-column MFMA tiles per wave
  constexpr int AROWS = kBlockM / kRowsPerPass; // A rows loaded per thread
  constexpr int BROWS = BN / kRowsPerPass;      // B rows loaded per thread
  constexpr int kTileBytes = (kBlockM + BN) * kRowBytes; // one stage
  constexpr int kLoads = AROWS + BROWS; // loads per producer thread and step
  extern __shared__ __align__(16) char lds[]; // NS * kTileBytes + row table
  // Per tile row: {byte offset of the input element under tap (0, 0), channel
  // 0 of the group; mask of taps that read inside the input}.
  uint2 *rowTable = reinterpret_cast<uint2 *>(lds + NS * kTileBytes);
  // ... and, where kernel taps are told apart by ranges and the field has a
  // depth, the range of valid kernel planes.
  uint32_t *depthTable = reinterpret_cast<uint32_t *>(rowTable + kBlockM);

  const IgemmDesc &d = a.d;
  // tile = ((part * groups + g) * mTiles + mTile) * nTiles + nTile, taken
  // apart with multiply-high divisions: a generic division is some forty
  // instructions, and every wave would run four of them before anything else.
  const uint32_t tile = xcdSwizzle(block, blocks);
  const uint32_t overN = a.divNTiles(tile);
  const uint32_t nTile = tile - overN * a.nTiles;
  const uint32_t gs = a.divMTiles(overN);
  const uint32_t mTile = overN - gs * a.mTiles;
  const uint32_t part = a.divGroups(gs); // which part of K
  const uint32_t g = gs - part * d.groups;
  out += size_t(part) * a.M * (d.groups * d.outChansPerGroup);
  const uint32_t mode = a.mode;
  // The input is addressed with 32-bit offsets from the first image the
  // tile reads - a tile's rows span few images, the whole tensor may be far
  // larger than 2^31 bytes.
  const uint32_t firstImage =
      a.divOutD(a.divOutH(a.divOutW(mTile * kBlockM)));

  const int t = threadIdx.x;
  const bool producer = t >= kThreads - kProducers; // waves 4-7
  const uint32_t inChans = d.groups * d.inChansPerGroup;
  const uint32_t ciBytes = d.inChansPerGroup * EB; // bytes of K per tap
  const uint32_t pixelBytes = inChans * EB;
  const uint32_t taps = d.kD * d.kH * d.kW;

  const int wave = (t >> 6) & 3, lane = t & 63;
  const int wm = wave >> 1, wn = wave & 1;
  floatx16 acc[2][TN];

  if (producer) {
    // The producers' address arithmetic shares each SIMD's issue port with a
    // consumer's MFMAs: let their (short) vector instructions go first.
    __builtin_amdgcn_s_setprio(3);
    const int pt = t - (kThreads - kProducers);
    // producer wave, as a scalar: what depends on it alone (LDS destinations
    // of the loads) is then formed by scalar instructions
    const int pw = __builtin_amdgcn_readfirstlane(pt >> 6);
    // Lane l of a load fills row position (l >> 3) of an 8-row block at chunk
    // position (l & 7).  This wave's blocks all have the parity of pw: in
    // odd blocks that position belongs to row (l >> 3) ^ 1; either way the
    // lane fetches chunk (l & 7) ^ (row & 7).
    const int rowInBlock = (lane >> 3) ^ (pw & 1);
    const int chunk = (lane & 7) ^ rowInBlock;
    // The buffer starts `shift` bytes before the tensor, as many as the
    // largest amount a padded window reaches above / left of an image, so
    // that the per-row offset below is never negative: the buffer unit adds
    // the vector and scalar offsets without wrapping.  Nothing in front of
    // the tensor is ever read (such taps are masked).
    const uint32_t shift =
        mode == kDilatedTaps
            ? 0u
            : ((uint32_t(d.padD > 0 ? d.padD : 0) * d.inH +
                uint32_t(d.padH > 0 ? d.padH : 0)) *
                   d.inW +
               uint32_t(d.padW > 0 ? d.padW : 0)) *
                  pixelBytes;
    const uint64_t skipped = uint64_t(firstImage) * a.imageBytes;
    const uint64_t left = a.inBytes - skipped + shift;
    const __amdgpu_buffer_rsrc_t inBuf =
        bufferOf(in + skipped - shift,
                 uint32_t(left < kOutOfRange - 1 ? left : kOutOfRange - 1));
    const __amdgpu_buffer_rsrc_t wBuf = bufferOf(w, a.wBytes);

    // Load r of this wave fills the 8-row block (r * 4 + pw) of the A tile.
    // Per A row (output pixel) of this thread: the byte offset (from the
    // shifted buffer start) of the input element under kernel tap (0, 0),
    // channel chunk `chunk`, and one bit per kernel tap telling whether that
    // tap reads inside the input - read from the row table further down, once
    // the weight loads, which need none of it, are on their way.
    uint32_t rowOff[AROWS], tapMask[AROWS];
    int originW[AROWS];                       // dilated input only
    uint32_t khLo[AROWS], khSpan[AROWS], kwLo[AROWS], kwSpan[AROWS]; // ranges
    uint32_t kdLo[AROWS], kdSpan[AROWS];

    uint32_t bOff[BROWS];
#pragma unroll
    for (int r = 0; r != BROWS; ++r)
      bOff[r] = ((g * a.coPadded + nTile * BN + (r * 4 + pw) * 8 + rowInBlock) *
                     a.kPadded) *
                    EB +
                chunk * 16;
    // Byte offset of the next k-step along a row of the packed weights; this
    // part of K starts kStart bytes in.
    const uint32_t kStart = part * a.kSteps * kRowBytes;
    uint32_t kByte = kStart;
    auto loadB = [&](uint32_t stage) {
      char *base = lds + stage * kTileBytes + pw * kLoadBytes;
      // The position along K travels in the scalar offset, which the range
      // check leaves out: the steps beyond K - whole-wave events - ask for an
      // out-of-range vector offset instead.
      if (kByte < a.kPadded * EB) {
#pragma unroll
        for (int r = 0; r != BROWS; ++r)
          loadToLds(wBuf,
                    (LdsPtr)(base + kBlockM * kRowBytes + r * 4 * kLoadBytes),
                    bOff[r], kByte);
      } else {
#pragma unroll
        for (int r = 0; r != BROWS; ++r)
          loadToLds(wBuf,
                    (LdsPtr)(base + kBlockM * kRowBytes + r * 4 * kLoadBytes),
                    kOutOfRange, 0);
      }
      kByte += kRowBytes;
    };

    // The whole schedule, written once for both ways of addressing the input
    // (a compile-time choice inside, so that neither loop carries the other's
    // branches).  NS - 1 k-steps are in flight; the oldest is waited for
    // before each barrier.  Start-up order: all weight loads, then (row table
    // ready) the input loads of step 0, the first barrier, the input loads of
    // the other stages; from then on input and weight loads of one k-step
    // together.
    auto produce = [&](auto modeTag) {
      constexpr int MODE = decltype(modeTag)::value;
      constexpr bool GEN = MODE == kDilatedTaps;
      // Position inside K of the input data loaded next.  UNI: (tap, byte
      // offset of the channel block inside the tap) of the whole k-step,
      // wave-uniform.  Otherwise the same pair for this thread's own 16-byte
      // chunk.
      uint32_t aByte = kStart + (UNI ? 0 : chunk * 16);
      uint32_t tap = a.divCiBytes(aByte);
      uint32_t ciOff = aByte - tap * ciBytes;
      // tap = (kd * kH + kh) * kW + kw
      uint32_t kRow = a.divKW(tap), kw = tap - kRow * d.kW;
      uint32_t kd = a.divKH(kRow), kh = kRow - kd * d.kH;
      auto advance = [&] {
        if constexpr (GEN) {
          // no loop, no branch: everything again from the byte position
          aByte += kRowBytes;
          tap = a.divCiBytes(aByte);
          ciOff = aByte - tap * ciBytes;
          kh = a.divKW(tap); // (no depth with a dilated input)
          kw = tap - kh * d.kW;
        } else if constexpr (!UNI) {
          // Per thread, so a loop would diverge; straight-line code instead,
          // as above, with the depth
          aByte += kRowBytes;
          tap = a.divCiBytes(aByte);
          ciOff = aByte - tap * ciBytes;
          kRow = a.divKW(tap);
          kw = tap - kRow * d.kW;
          kd = a.divKH(kRow);
          kh = kRow - kd * d.kH;
        } else {
          ciOff += kRowBytes;
          while (ciOff >= ciBytes) {
            ciOff -= ciBytes;
            ++tap;
            if (++kw == d.kW) {
              kw = 0;
              if (++kh == d.kH) {
                kh = 0;
                ++kd;
              }
            }
          }
        }
      };
      auto loadA = [&](uint32_t stage) {
        char *base = lds + stage * kTileBytes + pw * kLoadBytes;
        if constexpr (GEN) {
          // rowOff: the row's image and group; tapMask / originW: its window
          // origin (row, column) in zero-stuffed input coordinates.  The tap
          // reads input (origin + tap * dilation) / input dilation when that
          // is whole and inside [lo, hi).  A producer wave gets to issue a
          // vector instruction only every few cycles and pays dearly for a
          // taken branch, so this is straight-line code: selects, 24-bit
          // multiplies (the launcher checks the ranges), and the division by
          // the input dilation also when that is 1.
          const int khd = int(kh * d.dilH), kwd = int(kw * d.dilW);
          const uint32_t tapOk = tap < taps ? 1u : 0u;
          const uint32_t lane16 = ciOff + (UNI ? chunk * 16 : 0) - chunk * 16;
          const uint32_t rowBytes = d.inW * pixelBytes;
          const uint32_t spanH = d.hiH - d.loH, spanW = d.hiW - d.loW;
          // One step of the computation for all rows before the next one:
          // a lone wave waits several cycles for a result it has just
          // issued, so neighbouring instructions should not depend on each
          // other.
          int ihD[AROWS], iwD[AROWS];
          uint32_t ih[AROWS], iw[AROWS], ok[AROWS], off[AROWS];
#pragma unroll
          for (int r = 0; r != AROWS; ++r) {
            ihD[r] = int(tapMask[r]) + khd;
            iwD[r] = originW[r] + kwd;
          }
#pragma unroll
          for (int r = 0; r != AROWS; ++r) {
            ih[r] = a.divInDilH(uint32_t(ihD[r]));
            iw[r] = a.divInDilW(uint32_t(iwD[r]));
          }
#pragma unroll
          for (int r = 0; r != AROWS; ++r)
            ok[r] = tapOk & uint32_t((ihD[r] | iwD[r]) >= 0) &
                    uint32_t(__umul24(ih[r], d.inDilH) == uint32_t(ihD[r])) &
                    uint32_t(__umul24(iw[r], d.inDilW) == uint32_t(iwD[r])) &
                    uint32_t(ih[r] - d.loH < spanH) &
                    uint32_t(iw[r] - d.loW < spanW);
#pragma unroll
          for (int r = 0; r != AROWS; ++r)
            off[r] = rowOff[r] + __umul24(ih[r], rowBytes) +
                     __umul24(iw[r], pixelBytes) + lane16;
#pragma unroll
          for (int r = 0; r != AROWS; ++r) {
            LdsPtr dst = (LdsPtr)(base + r * 4 * kLoadBytes);
            loadToLds(inBuf, dst, ok[r] ? off[r] : kOutOfRange, 0);
          }
        } else {
          const uint32_t tapOff =
              ((kd * d.dilD * d.inH + kh * d.dilH) * d.inW + kw * d.dilW) *
              pixelBytes;
          if constexpr (UNI && MODE == kMaskTaps) {
            // tapMask holds the complement of the row's mask here: shifted so
            // that the tap's bit lands on bit 31 and merged into the offset,
            // it makes the offset out of range exactly when the tap reads
            // padding - two vector instructions per row.
            if (tap < taps) {
              const uint32_t shiftToTop = 31 - tap;
#pragma unroll
              for (int r = 0; r != AROWS; ++r) {
                LdsPtr dst = (LdsPtr)(base + r * 4 * kLoadBytes);
                loadToLds(inBuf, dst,
                          (rowOff[r] & 0x7fffffffu) |
                              ((tapMask[r] << shiftToTop) & 0x80000000u),
                          tapOff + ciOff);
              }
            } else {
#pragma unroll
              for (int r = 0; r != AROWS; ++r)
                loadToLds(inBuf, (LdsPtr)(base + r * 4 * kLoadBytes),
                          kOutOfRange, 0);
            }
            advance();
            return;
          }
          const uint32_t tapBit = tap < taps ? (1u << (tap & 31)) : 0u;
#pragma unroll
          for (int r = 0; r != AROWS; ++r) {
            bool ok;
            if constexpr (MODE == kRangeTaps)
              ok = (tap < taps) & (kh - khLo[r] < khSpan[r]) &
                   (kw - kwLo[r] < kwSpan[r]) & (kd - kdLo[r] < kdSpan[r]);
            else
              ok = (tapMask[r] & tapBit) != 0;
            LdsPtr dst = (LdsPtr)(base + r * 4 * kLoadBytes);
            if constexpr (UNI)
              loadToLds(inBuf, dst, ok ? rowOff[r] : kOutOfRange,
                        tapOff + ciOff);
            else
              loadToLds(inBuf, dst,
                        ok ? rowOff[r] - chunk * 16 + tapOff + ciOff
                           : kOutOfRange,
                        0);
          }
        }
        advance();
      };
#pragma unroll
      for (int r = 0; r != AROWS; ++r) {
        const uint2 e = rowTable[(r * 4 + pw) * 8 + rowInBlock];
        rowOff[r] = e.x + chunk * 16;
        tapMask[r] = GEN ? uint32_t(int(e.y >> 16) - 32768)
                     : UNI && MODE == kMaskTaps ? ~e.y
                                                : e.y;
        originW[r] = int(e.y & 0xffffu) - 32768;
        if constexpr (MODE == kRangeTaps) {
          // columns: 16 bits a piece; rows and planes: 8 bits a piece
          kwLo[r] = e.y & 0xffffu, kwSpan[r] = e.y >> 16;
          const uint32_t planes = depthTable[(r * 4 + pw) * 8 + rowInBlock];
          khLo[r] = planes & 0xffu, khSpan[r] = (planes >> 8) & 0xffu;
          kdLo[r] = (planes >> 16) & 0xffu, kdSpan[r] = planes >> 24;
        } else {
          khLo[r] = kwLo[r] = kdLo[r] = 0;
          khSpan[r] = kwSpan[r] = kdSpan[r] = 1;
        }
      }
      // The consumers start as soon as step 0 is there; the input loads of
      // the other stages go out behind their back.
      loadA(0);
      MXK_WAIT_VMCNT(0);
      stepBarrier(); // barrier 0: step 0 is in LDS stage 0
#pragma unroll
      for (int s = 1; s != NS - 1; ++s)
        loadA(s);
      for (uint32_t kt = 0; kt != a.kSteps; ++kt) {
        // Stage (kt - 1) % NS was multiplied before the last barrier: refill
        // it with step kt + NS - 1, then make sure step kt + 1 has landed.
        // The first time round the start-up order still shows in the queue.
        loadA((kt + NS - 1) % NS);
        loadB((kt + NS - 1) % NS);
        if (kt == 0 && NS > 2)
          MXK_WAIT_VMCNT((NS - 3) * AROWS + kLoads);
        else
          MXK_WAIT_VMCNT((NS - 2) * kLoads);
        stepBarrier(); // barrier kt + 1
      }
    };

#pragma unroll
    for (int s = 0; s != NS - 1; ++s)
      loadB(s);
    stepBarrier(); // the row table is complete
    if (mode == kDilatedTaps)
      produce(std::integral_constant<int, kDilatedTaps>{});
    else if (mode == kRangeTaps)
      produce(std::integral_constant<int, kRangeTaps>{});
    else
      produce(std::integral_constant<int, kMaskTaps>{});
    MXK_WAIT_VMCNT(0); // the trailing zero loads, before LDS is reused
  } else {
    // While the producers start the weight loads, the first 128 consumer
    // threads work out the row table, one tile row each.
    if (t < kBlockM) {
      const uint32_t m = mTile * kBlockM + t;
      const bool rowValid = m < a.M;
      const uint32_t mm = rowValid ? m : 0;
      const uint32_t q = a.divOutW(mm);
      const uint32_t ow = mm - q * d.outW;
      const uint32_t q2 = a.divOutH(q);
      const uint32_t oh = q - q2 * d.outH;
      const uint32_t image = a.divOutD(q2);
      const uint32_t od = q2 - image * d.outD;
      const uint32_t b = image - firstImage; // (0 for an invalid row: unused)
      const int idBase = int(od * d.strideD) - d.padD;
      const int ihBase = int(oh * d.strideH) - d.padH;
      const int iwBase = int(ow * d.strideW) - d.padW;
      const uint32_t shift = ((uint32_t(d.padD > 0 ? d.padD : 0) * d.inH +
                               uint32_t(d.padH > 0 ? d.padH : 0)) *
                                  d.inW +
                              uint32_t(d.padW > 0 ? d.padW : 0)) *
                             pixelBytes;
      // byte offset of the input element under tap (0, 0, 0) from the
      // (shifted) buffer start; the additions wrap where a window starts
      // above or left of the image and come right again with the shift
      const uint32_t originOffset =
          shift +
          (((b * d.inD + uint32_t(idBase)) * d.inH + uint32_t(ihBase)) *
               d.inW +
           uint32_t(iwBase)) *
              pixelBytes +
          g * ciBytes;
      if (mode == kDilatedTaps) {
        // An invalid row gets the origin (-32768, -32768): no tap of it is
        // ever inside the input.
        rowTable[t] = uint2{
            b * d.inH * d.inW * pixelBytes + g * ciBytes,
            rowValid ? (uint32_t(ihBase + 32768) << 16) |
                           uint32_t(iwBase + 32768)
                     : 0u};
      } else if (mode == kRangeTaps) {
        // Kernel rows kh with lo <= base + kh * dilation < hi form an
        // interval; so do the columns and the planes.  {first, length} of
        // each: the columns' in 16 bits a piece (the kernel of a 1-D layer's
        // weight update pass is as long as the layer's output), the others'
        // in 8; an invalid row gets an empty interval of columns.
        auto range = [](int base, int lo, int hi, int dil, int size,
                        int bits) {
          auto ceilDiv = [](int n, int dv) {
            return n >= 0 ? (n + dv - 1) / dv : -((-n) / dv);
          };
          int first = ceilDiv(lo - base, dil), last = ceilDiv(hi - base, dil);
          first = first < 0 ? 0 : first > size ? size : first;
          last = last < first ? first : last > size ? size : last;
          return uint32_t(first) | (uint32_t(last - first) << bits);
        };
        const uint32_t columns =
            range(iwBase, int(d.loW), int(d.hiW), int(d.dilW), int(d.kW), 16);
        rowTable[t] = uint2{originOffset, rowValid ? columns : 0u};
        depthTable[t] =
            range(ihBase, int(d.loH), int(d.hiH), int(d.dilH), int(d.kH), 8) |
            (range(idBase, int(d.loD), int(d.hiD), int(d.dilD), int(d.kD), 8)
             << 16);
      } else {
        uint32_t mask = 0;
        if (d.dilD == 1 && d.dilH == 1 && d.dilW == 1) {
          // Undilated kernel: the valid kernel columns are the interval
          // [lo - base, hi - base) cut to the kernel, and so are the rows.
          // Bits [first, last) of a word:
          auto bitRange = [](int first, int last) {
            return first < last ? uint32_t(((1ull << last) - 1) &
                                           ~((1ull << first) - 1))
                                : 0u;
          };
          auto cut = [](int v, int size) {
            return v < 0 ? 0 : v > size ? size : v;
          };
          const int kW = int(d.kW), kH = int(d.kH), kD = int(d.kD);
          const uint32_t kwMask = bitRange(cut(int(d.loW) - iwBase, kW),
                                           cut(int(d.hiW) - iwBase, kW));
          // one bit per valid kernel row, at that row's first tap; the
          // product puts the column mask there (no carries: it is narrower
          // than the distance between the bits)
          const uint32_t rowStarts =
              a.tapRowStarts & bitRange(cut(int(d.loH) - ihBase, kH) * kW,
                                        cut(int(d.hiH) - ihBase, kH) * kW);
          // likewise one bit per valid kernel plane, at its first tap
          const uint32_t planeStarts =
              a.tapPlaneStarts &
              bitRange(cut(int(d.loD) - idBase, kD) * kH * kW,
                       cut(int(d.hiD) - idBase, kD) * kH * kW);
          mask = kwMask * rowStarts * planeStarts;
        } else {
          uint32_t kwMask = 0;
          for (uint32_t kw = 0; kw != d.kW; ++kw) {
            const int iw = iwBase + int(kw * d.dilW);
            if (iw >= int(d.loW) && iw < int(d.hiW))
              kwMask |= 1u << kw;
          }
          uint32_t planeMask = 0;
          for (uint32_t kh = 0; kh != d.kH; ++kh) {
            const int ih = ihBase + int(kh * d.dilH);
            if (ih >= int(d.loH) && ih < int(d.hiH))
              planeMask |= kwMask << (kh * d.kW);
          }
          for (uint32_t kd = 0; kd != d.kD; ++kd) {
            const int id = idBase + int(kd * d.dilD);
            if (id >= int(d.loD) && id < int(d.hiD))
              mask |= planeMask << (kd * d.kH * d.kW);
          }
        }
        rowTable[t] = uint2{originOffset, rowValid ? mask : 0u};
      }
    }
    MXK_WAIT_LGKMCNT0();
    stepBarrier(); // the row table is complete
#pragma unroll
    for (int i = 0; i != 2; ++i)
#pragma unroll
      for (int j = 0; j != TN; ++j)
#pragma unroll
        for (int v = 0; v != 16; ++v)
          acc[i][j][v] = 0.0f;
    using M = Mma<EB>;
    constexpr int SS = M::kSubSteps;
    constexpr int P = SS / 2; // sub-steps fetched ahead
    typename M::template Frags<TN> f;
    // Instructions may not be moved across this point: the order written
    // here - which LDS reads are in flight under which MFMAs - is the
    // software pipeline.
    auto pin = [] { __builtin_amdgcn_sched_barrier(0); };
    const int rowOffset = fragmentRowOffset(lane);
    auto fetch = [&](uint32_t kt, auto sub) {
      const char *stage = lds + (kt % NS) * kTileBytes;
      const char *tileA = stage + wm * 64 * kRowBytes + rowOffset;
      const FragmentAddress at{
          {tileA, tileA + 32 * kRowBytes},
          {lane & 7, lane & 7},
          0,
          stage + (kBlockM + wn * (BN / 2)) * kRowBytes + rowOffset,
          lane & 7};
      M::template load<decltype(sub)::value, TN>(at, lane, f);
    };
    // Sub-steps [0, P) of a k-step are fetched during the previous k-step,
    // sub-step s + P under the MFMAs of sub-step s.  The workgroup barrier
    // sits before the last sub-step: every LDS read of this stage has
    // returned by then (the producers may refill it), the next stage has
    // landed, and its first reads go out under the last sub-step's MFMAs.
    stepBarrier(); // barrier 0
    if (a.kSteps != 0)
      staticFor<0, P>([&](auto sub) { fetch(0, sub); });
    pin();
    for (uint32_t kt = 0; kt != a.kSteps; ++kt) {
      staticFor<0, SS - 1>([&](auto sub) {
        constexpr int S = decltype(sub)::value;
        M::template mul<S, TN, FA, FB>(f, acc, [&] {
          if constexpr (S + P < SS)
            fetch(kt, std::integral_constant<int, S + P>{});
        });
        pin();
      });
      MXK_WAIT_LGKMCNT0();
      stepBarrier(); // barrier kt + 1: step kt + 1 has landed
      pin();
      M::template mul<SS - 1, TN, FA, FB>(f, acc, [&] {
        if (kt + 1 != a.kSteps)
          staticFor<0, P>([&](auto sub) { fetch(kt + 1, sub); });
      });
      pin();
    }
  }
  // One more meeting point: the producers' trailing loads have landed, so
  // LDS can be reused for the output tile.
  __syncthreads();

  static_assert(epilogueLdsBytes<BN, OutT>() <=
                    igemmLdsBytes<BN, NS, OutT>(),
                "epilogue tile fits LDS");
  igemmEpilogue<BN, OutT>(lds, a, acc, producer, t, lane, wm, wn, mTile, nTile,
                          g, bias, out, scale);
}

template <int BN, int NS, int EB, int FA, int FB, bool UNI, class OutT>
__global__ __launch_bounds__(kThreads) void igemmKernel(
    IgemmArgs a, const char *__restrict__ in, const char *__restrict__ w,
    const OutT *__restrict__ bias, OutT *__restrict__ out, float scale) {
  igemmTile<BN, NS, EB, FA, FB, UNI, OutT>(a, in, w, bias, out, scale,
                                           blockIdx.x, gridDim.x);
}

/// Several convolutions that run the same kernel, in one launch: the grid is
/// the concatenation of their tiles, so that convolutions too small to fill
/// the chip share it.  (PopLibs' parallel multi-convolution plan gives each
/// a disjoint range of tiles, lib/poplin/MultiConvolution.cpp:125-176.)
constexpr int kMaxFused = int(kIgemmMaxFused);
struct IgemmFusedArgs {
  uint32_t count;
  uint32_t firstBlock[kMaxFused + 1]; // prefix sums of the tile counts
  IgemmArgs a[kMaxFused];
  const char *in[kMaxFused];
  const char *w[kMaxFused];
  const void *bias[kMaxFused];
  void *out[kMaxFused];
  float scale[kMaxFused];
};

template <int BN, int NS, int EB, int FA, int FB, bool UNI, class OutT>
__global__ __launch_bounds__(kThreads) void igemmFusedKernel(IgemmFusedArgs m) {
  uint32_t i = 0;
  while (i + 1 < m.count && blockIdx.x >= m.firstBlock[i + 1])
    ++i;
  igemmTile<BN, NS, EB, FA, FB, UNI, OutT>(
      m.a[i], m.in[i], m.w[i], static_cast<const OutT *>(m.bias[i]),
      static_cast<OutT *>(m.out[i]), m.scale[i], blockIdx.x - m.firstBlock[i],
      m.firstBlock[i + 1] - m.firstBlock[i]);
}

template <class Kernel>
hipError_t raiseLdsLimit(Kernel kernel, int ldsBytes) {
  // More than the 64 KB a kernel gets by default.
  return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize,
                             ldsBytes);
}

/// What to launch once the kernel's template arguments are known: one
/// convolution ...
struct LaunchOne {
  const IgemmArgs &a;
  const void *in, *w, *bias;
  void *out;
  float scale;
  hipStream_t stream;
  template <int BN, int NS, int EB, int FA, int FB, bool UNI, class OutT>
  hipError_t go() const {
    const uint64_t blocks =
        uint64_t(a.mTiles) * a.nTiles * a.d.groups * a.d.splitK;
    if (blocks == 0)
      return hipSuccess;
    if (blocks > 0x7fffffffull)
      return hipErrorInvalidConfiguration;
    constexpr int ldsBytes = igemmLdsBytes<BN, NS, OutT>();
    static const hipError_t attr = raiseLdsLimit(
        &igemmKernel<BN, NS, EB, FA, FB, UNI, OutT>, ldsBytes);
    if (attr != hipSuccess)
      return attr;
    hipLaunchKernelGGL((igemmKernel<BN, NS, EB, FA, FB, UNI, OutT>),
                       dim3(uint32_t(blocks)), dim3(kThreads), ldsBytes,
                       stream, a, static_cast<const char *>(in),
                       static_cast<const char *>(w),
                       static_cast<const OutT *>(bias),
                       static_cast<OutT *>(out), scale);
    return hipGetLastError();
  }
};

/// ... or several in one grid.
struct LaunchFused {
  const IgemmFusedArgs &m;
  hipStream_t stream;
  template <int BN, int NS, int EB, int FA, int FB, bool UNI, class OutT>
  hipError_t go() const {
    const uint32_t blocks = m.firstBlock[m.count];
    if (blocks == 0)
      return hipSuccess;
    constexpr int ldsBytes = igemmLdsBytes<BN, NS, OutT>();
    static const hipError_t attr = raiseLdsLimit(
        &igemmFusedKernel<BN, NS, EB, FA, FB, UNI, OutT>, ldsBytes);
    if (attr != hipSuccess)
      return attr;
    hipLaunchKernelGGL((igemmFusedKernel<BN, NS, EB, FA, FB, UNI, OutT>),
                       dim3(blocks), dim3(kThreads), ldsBytes, stream, m);
    return hipGetLastError();
  }
};

/// The kernel instantiation a convolution runs.
struct KernelKey {
  int blockN, stages, inType, outType, fa, fb;
  bool uni;
  bool operator==(const KernelKey &o) const {
    return blockN == o.blockN && stages == o.stages && inType == o.inType &&
           outType == o.outType && fa == o.fa && fb == o.fb && uni == o.uni;
  }
};

KernelKey kernelKey(const IgemmDesc &d, int inType, int outType,
                    const QuarterInfo &q) {
  const int eb = inType == kFloat ? 4 : inType == kHalf ? 2 : 1;
  KernelKey k;
  k.blockN = int(d.blockN), k.inType = inType, k.outType = outType;
  k.stages = d.blockN == 128 ? int(d.stages) : 3;
  // Instruction format codes: 0 = E4M3, 1 = E5M2.
  k.fa = inType == kQuarter && q.inFormat != kE4M3 ? 1 : 0;
  k.fb = inType == kQuarter && q.weightFormat != kE4M3 ? 1 : 0;
  k.uni = (d.inChansPerGroup * eb) % kRowBytes == 0;
  return k;
}

template <int BN, int NS, int EB, int FA, int FB, class Launch>
hipError_t dispatchOut(const KernelKey &k, const Launch &launch) {
  if (k.outType == kHalf)
    return k.uni
               ? launch.template go<BN, NS, EB, FA, FB, true, __half>()
               : launch.template go<BN, NS, EB, FA, FB, false, __half>();
  if (k.outType == kFloat)
    return k.uni ? launch.template go<BN, NS, EB, FA, FB, true, float>()
                 : launch.template go<BN, NS, EB, FA, FB, false, float>();
  return hipErrorInvalidValue;
}

template <int BN, int EB, int FA, int FB, class Launch>
hipError_t dispatchStages(const KernelKey &k, const Launch &launch) {
  // Stages of LDS.  128-wide tile: 4 x 32 KB (one workgroup per CU) or
  // 2 x 32 KB (two per CU); 64-wide tile: 3 x 24 KB (two per CU).
  if constexpr (BN == 128) {
    if (k.stages == 4)
      return dispatchOut<BN, 4, EB, FA, FB>(k, launch);
    if (k.stages == 2)
      return dispatchOut<BN, 2, EB, FA, FB>(k, launch);
    return hipErrorInvalidValue;
  } else {
    return dispatchOut<BN, 3, EB, FA, FB>(k, launch);
  }
}

template <int BN, class Launch>
hipError_t dispatchType(const KernelKey &k, const Launch &launch) {
  if (k.inType == kHalf)
    return dispatchStages<BN, 2, 0, 0>(k, launch);
  if (k.inType == kFloat)
    return dispatchStages<BN, 4, 0, 0>(k, launch);
  if (k.inType != kQuarter)
    return hipErrorInvalidValue;
  if (k.fa == 0 && k.fb == 0)
    return dispatchStages<BN, 1, 0, 0>(k, launch);
  if (k.fa == 0 && k.fb == 1)
    return dispatchStages<BN, 1, 0, 1>(k, launch);
  if (k.fa == 1 && k.fb == 0)
    return dispatchStages<BN, 1, 1, 0>(k, launch);
  return dispatchStages<BN, 1, 1, 1>(k, launch);
}

template <class Launch>
hipError_t dispatch(const KernelKey &k, const Launch &launch) {
  if (k.blockN == 128)
    return dispatchType<128>(k, launch);
  if (k.blockN == 64)
    return dispatchType<64>(k, launch);
  return hipErrorInvalidValue;
}

/// out[i] = sum over parts of partial[part][i] (+ bias of i's channel).  The
/// parts are added in a fixed order: four interleaved running sums (so that
/// four loads are in flight per lane), combined at the end.  A thread takes V
/// neighbouring channels of one pixel: 4 where the channel count is a multiple
/// of 4 (one 16-byte load per part), else 1.
template <class OutT, int V>
__global__ __launch_bounds__(64) void splitKReduceKernel(
    const float *__restrict__ partial, uint32_t parts, uint64_t elems,
    uint32_t channels, const OutT *__restrict__ bias, OutT *__restrict__ out,
    bool transposed) {
  const uint64_t i = (uint64_t(blockIdx.x) * blockDim.x + threadIdx.x) * V;
  if (i >= elems)
    return;
  float sum[4][V] = {};
  const auto add = [&](int u, uint32_t part) {
    const float *src = partial + uint64_t(part) * elems + i;
    if constexpr (V == 4) {
      const float4 v = *reinterpret_cast<const float4 *>(src);
      sum[u][0] += v.x, sum[u][1] += v.y, sum[u][2] += v.z, sum[u][3] += v.w;
    } else {
      sum[u][0] += *src;
    }
  };
  uint32_t p = 0;
  for (; p + 4 <= parts; p += 4) {
#pragma unroll
    for (int u = 0; u != 4; ++u)
      add(u, p + u);
  }
  for (; p != parts; ++p)
    add(0, p);
  float v[V];
#pragma unroll
  for (int e = 0; e != V; ++e)
    v[e] = (sum[0][e] + sum[1][e]) + (sum[2][e] + sum[3][e]);
  const uint32_t c = uint32_t(i % channels);
  if (bias) {
#pragma unroll
    for (int e = 0; e != V; ++e)
      v[e] += Load<OutT>::at(bias, c + e, 0);
  }
  if (transposed) {
    // [channel][pixel]
    const uint64_t pixels = elems / channels, pixel = i / channels;
#pragma unroll
    for (int e = 0; e != V; ++e)
      storeOut(out, (c + e) * pixels + pixel, v[e]);
    return;
  }
  if constexpr (V == 4)
    storeOut4(out + i, v);
  else
    storeOut(out, i, v[0]);
}

template <class OutT>
void launchSplitKReduce(const float *partial, uint32_t parts, uint64_t elems,
                        uint32_t channels, const void *bias, void *out,
                        bool transposed, hipStream_t stream) {
  const int v = channels % 4 == 0 ? 4 : 1;
  const uint32_t blocks = uint32_t((elems / v + 63) / 64);
  if (v == 4)
    hipLaunchKernelGGL((splitKReduceKernel<OutT, 4>), dim3(blocks), dim3(64),
                       0, stream, partial, parts, elems, channels,
                       static_cast<const OutT *>(bias),
                       static_cast<OutT *>(out), transposed);
  else
    hipLaunchKernelGGL((splitKReduceKernel<OutT, 1>), dim3(blocks), dim3(64),
                       0, stream, partial, parts, elems, channels,
                       static_cast<const OutT *>(bias),
                       static_cast<OutT *>(out), transposed);
}

} // namespace

int igemmTapAddressing(const IgemmDesc &d) {
  if (d.inDilH != 1 || d.inDilW != 1)
    return kDilatedTaps;
  return d.kD * d.kH * d.kW > 32 ? kRangeTaps : kMaskTaps;
}

bool igemmAddressable(const IgemmDesc &d, int inType) {
  const uint64_t eb = inType == kFloat ? 4 : inType == kHalf ? 2 : 1;
  const uint64_t imageBytes =
      uint64_t(d.inD) * d.inH * d.inW * d.groups * d.inChansPerGroup * eb;
  const uint64_t shift = ((uint64_t(d.padD > 0 ? d.padD : 0) * d.inH +
                           uint64_t(d.padH > 0 ? d.padH : 0)) *
                              d.inW +
                          uint64_t(d.padW > 0 ? d.padW : 0)) *
                         d.groups * d.inChansPerGroup * eb;
  // images a tile of 128 output rows can touch: its rows' own, one more when
  // it starts inside an image
  const uint64_t rowsPerImage = uint64_t(d.outD) * d.outH * d.outW;
  if (rowsPerImage == 0)
    return true;
  uint64_t images = (kBlockM - 1) / rowsPerImage + 2;
  if (images > d.batch)
    images = d.batch;
  return images * imageBytes + shift < kOutOfRange - (1u << 20);
}

size_t igemmWorkspaceBytes(const IgemmDesc &d) {
  if (d.splitK <= 1)
    return 0;
  return size_t(d.splitK) * d.batch * d.outD * d.outH * d.outW * d.groups *
         d.outChansPerGroup * sizeof(float);
}

namespace {

/// Checks `d` against what the kernels are compiled for (the planner only
/// produces such shapes) and fills in the kernel's arguments.
hipError_t prepare(const IgemmDesc &d, int inType, bool haveWorkspace,
                   IgemmArgs &a) {
  const uint32_t eb = inType == kFloat ? 4 : inType == kHalf ? 2 : 1;
  const uint32_t bke = kRowBytes / eb;
  const int mode = igemmTapAddressing(d);
  const bool dilated = mode == kDilatedTaps;
  if (d.blockM != kBlockM || (d.blockN != 64 && d.blockN != 128) ||
      d.blockK != bke || d.inChansPerGroup % (16 / eb) != 0 ||
      (inType != kHalf && inType != kQuarter && inType != kFloat) ||
      d.splitK == 0 ||
      d.inDilH == 0 || d.inDilW == 0)
    return hipErrorInvalidValue;
  // The arithmetic addressing keeps window origins as 16-bit offsets from
  // -32768 and never reaches a tap beyond +32767 of them; its
  // multiplications are 24-bit ones.
  if (dilated &&
      (uint64_t(d.outH) * d.strideH + uint64_t(d.kH) * d.dilH +
               uint64_t(d.padH > 0 ? d.padH : -d.padH) >=
           32768 ||
       uint64_t(d.outW) * d.strideW + uint64_t(d.kW) * d.dilW +
               uint64_t(d.padW > 0 ? d.padW : -d.padW) >=
           32768 ||
       uint64_t(d.inW) * d.groups * d.inChansPerGroup * eb >= (1u << 24) ||
       d.inH >= (1u << 24) || d.inDilH >= (1u << 24) ||
       d.inDilW >= (1u << 24)))
    return hipErrorInvalidValue;
  // the ranges of valid kernel rows are kept in 8 bits a piece, of columns
  // in 16
  if (mode == kRangeTaps && (d.kH > 255 || d.kW > 32767))
    return hipErrorInvalidValue;
  // a depth dimension goes with the tap mask and the ranges
  if (mode == kDilatedTaps && (d.inD != 1 || d.outD != 1 || d.kD != 1))
    return hipErrorInvalidValue;
  if (mode == kRangeTaps && d.kD > 255)
    return hipErrorInvalidValue;
  if (d.kD == 0 || d.kH == 0 || d.kW == 0)
    return hipErrorInvalidValue;
  // outputs mapped into a larger field: plain 2-D convolutions, K not split
  const bool outMapped = d.outFullH != 0 || d.outFullW != 0;
  const uint32_t fullD = d.outFullD ? d.outFullD : d.outD;
  if (outMapped &&
      (d.splitK != 1 || d.outStepH == 0 || d.outStepW == 0 ||
       d.outStepD == 0 ||
       (d.outD != 0 && (d.outD - 1) * d.outStepD + d.outOffD >= fullD) ||
       (d.outH != 0 && (d.outH - 1) * d.outStepH + d.outOffH >= d.outFullH) ||
       (d.outW != 0 && (d.outW - 1) * d.outStepW + d.outOffW >= d.outFullW)))
    return hipErrorInvalidValue;
  if (d.splitK > 1 && !haveWorkspace)
    return hipErrorInvalidValue;
  a.d = d;
  a.d.outFullD = fullD;
  a.mode = uint32_t(mode);
  a.outMapped = outMapped ? 1u : 0u;
  if (d.outTransposed && outMapped)
    return hipErrorInvalidValue;
  // (with K split the workgroups write partial tiles, [pixel][channel] as
  // ever; the kernel that adds them up transposes)
  a.outTransposed = d.outTransposed && d.splitK == 1 ? 1u : 0u;
  a.divInDilH = makeFastDiv(d.inDilH);
  a.divInDilW = makeFastDiv(d.inDilW);
  a.divCiBytes = makeFastDiv(d.inChansPerGroup * eb);
  a.divKW = makeFastDiv(d.kW);
  a.divKH = makeFastDiv(d.kH);
  const uint64_t m = uint64_t(d.batch) * d.outD * d.outH * d.outW;
  if (m > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  a.M = uint32_t(m);
  a.divOutW = makeFastDiv(d.outW);
  a.divOutH = makeFastDiv(d.outH);
  a.divOutD = makeFastDiv(d.outD);
  a.mTiles = (a.M + kBlockM - 1) / kBlockM;
  a.nTiles = (d.outChansPerGroup + d.blockN - 1) / d.blockN;
  a.divNTiles = makeFastDiv(a.nTiles);
  a.divMTiles = makeFastDiv(a.mTiles);
  a.divGroups = makeFastDiv(d.groups);
  // bit kh * kW for every kernel row (tap mask mode: at most 32 taps)
  a.tapRowStarts = a.tapPlaneStarts = 0;
  if (a.mode == kMaskTaps) {
    for (uint32_t kh = 0; kh != d.kH; ++kh)
      a.tapRowStarts |= 1u << (kh * d.kW);
    for (uint32_t kd = 0; kd != d.kD; ++kd)
      a.tapPlaneStarts |= 1u << (kd * d.kH * d.kW);
  }
  a.coPadded = a.nTiles * d.blockN;
  const uint32_t k = d.kD * d.kH * d.kW * d.inChansPerGroup;
  a.kPadded = (k + bke - 1) / bke * bke;
  // every part runs the same number of k-steps; steps beyond K load zeros
  a.kSteps = d.noTaps ? 0 : (a.kPadded / bke + d.splitK - 1) / d.splitK;
  // Buffer addressing is 32-bit: the weights as a whole, the input from the
  // first image a tile reads (igemmAddressable; the planner keeps other
  // shapes away).
  const uint64_t wBytes = uint64_t(d.groups) * a.coPadded * a.kPadded * eb;
  if (!igemmAddressable(d, inType) || wBytes >= kOutOfRange)
    return hipErrorInvalidConfiguration;
  a.imageBytes = uint32_t(uint64_t(d.inD) * d.inH * d.inW * d.groups *
                          d.inChansPerGroup * eb);
  a.inBytes = uint64_t(d.batch) * a.imageBytes;
  a.wBytes = uint32_t(wBytes);
  return hipSuccess;
}

} // namespace

hipError_t launchIgemm(const IgemmDesc &d, int inType, int outType,
                       const void *in, const void *weightsPacked,
                       const void *bias, void *out, void *workspace,
                       const QuarterInfo &q, hipStream_t stream) {
  IgemmArgs a;
  hipError_t e = prepare(d, inType, workspace != nullptr, a);
  if (e != hipSuccess)
    return e;
  const float scale = inType == kQuarter ? q.scale : 1.0f;
  if (d.splitK == 1)
    return dispatch(kernelKey(d, inType, outType, q),
                    LaunchOne{a, in, weightsPacked, bias, out, scale, stream});
  // fp32 partial tiles per part (scaled, without bias), then their sum.
  e = dispatch(kernelKey(d, inType, kFloat, q),
               LaunchOne{a, in, weightsPacked, nullptr, workspace, scale,
                         stream});
  if (e != hipSuccess)
    return e;
  const uint32_t channels = d.groups * d.outChansPerGroup;
  const uint64_t elems = uint64_t(a.M) * channels;
  if (elems == 0)
    return hipSuccess;
  if ((elems + 63) / 64 > 0x7fffffffull)
    return hipErrorInvalidConfiguration;
  const float *partial = static_cast<const float *>(workspace);
  if (outType == kHalf)
    launchSplitKReduce<__half>(partial, d.splitK, elems, channels, bias, out,
                               d.outTransposed != 0, stream);
  else if (outType == kFloat)
    launchSplitKReduce<float>(partial, d.splitK, elems, channels, bias, out,
                              d.outTransposed != 0, stream);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

bool igemmFusable(const IgemmFusedItem &x, const IgemmFusedItem &y) {
  return x.d->splitK == 1 && y.d->splitK == 1 &&
         kernelKey(*x.d, x.inType, x.outType, x.q) ==
             kernelKey(*y.d, y.inType, y.outType, y.q);
}

hipError_t launchIgemmFused(const IgemmFusedItem *items, size_t count,
                            hipStream_t stream) {
  if (count == 0)
    return hipSuccess;
  if (count > size_t(kMaxFused))
    return hipErrorInvalidValue;
  IgemmFusedArgs m{};
  m.count = uint32_t(count);
  uint64_t blocks = 0;
  for (size_t i = 0; i != count; ++i) {
    const IgemmFusedItem &x = items[i];
    if (!igemmFusable(items[0], x))
      return hipErrorInvalidValue;
    const hipError_t e = prepare(*x.d, x.inType, false, m.a[i]);
    if (e != hipSuccess)
      return e;
    m.firstBlock[i] = uint32_t(blocks);
    blocks += uint64_t(m.a[i].mTiles) * m.a[i].nTiles * x.d->groups;
    if (blocks > 0x7fffffffull)
      return hipErrorInvalidConfiguration;
    m.in[i] = static_cast<const char *>(x.in);
    m.w[i] = static_cast<const char *>(x.weightsPacked);
    m.bias[i] = x.bias;
    m.out[i] = x.out;
    m.scale[i] = x.inType == kQuarter ? x.q.scale : 1.0f;
  }
  m.firstBlock[count] = uint32_t(blocks);
  return dispatch(kernelKey(*items[0].d, items[0].inType, items[0].outType,
                            items[0].q),
                  LaunchFused{m, stream});
}

} // namespace mxk

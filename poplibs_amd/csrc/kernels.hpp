// Host-callable launchers of the gfx950 kernels and the plain-data
// descriptors they take.  Everything here is independent of the ConvParams
// C++ class so that the kernels see only what they need.
#ifndef poplibs_amd_kernels_hpp
#define poplibs_amd_kernels_hpp
#include <cstddef>
#include <cstdint>
#include <hip/hip_runtime_api.h>

namespace mxk {

constexpr int kMaxDims = 4;

// Element type ids shared with the C ABI (mxconv_type).
enum : int { kQuarter = 0, kHalf = 1, kFloat = 2 };
// FP8 encodings (bit 7 of a quarter metadata byte).
enum : int { kE5M2 = 0, kE4M3 = 1 };

/// One spatial dimension of an input or kernel transform.
struct DimTransform {
  uint32_t size, truncLo, truncHi, dilation, padLo, padHi, flip;
  uint32_t transformedSize; // padLo + dilated(size - truncLo - truncHi) + padHi
};

/// Everything the any-parameter direct kernel needs.
struct GenericDesc {
  uint32_t numDims;
  uint32_t batch, groups, inChansPerGroup, outChansPerGroup;
  DimTransform in[kMaxDims];
  DimTransform kernel[kMaxDims];
  uint32_t outSize[kMaxDims];
  uint32_t outTruncLo[kMaxDims], outStride[kMaxDims];
  uint32_t outPadLo[kMaxDims], outPadHi[kMaxDims];
  uint32_t kernelElems; // product of kernel sizes
  uint64_t outElems;    // batch * prod(outSize) * groups * outChansPerGroup
};

/// Quarter (FP8) operands: encodings and the combined power-of-two scale.
struct QuarterInfo {
  int inFormat = kE4M3, weightFormat = kE4M3;
  float scale = 1.0f; // 2^(scaleIn + scaleWeights)
};

/// Any ConvParams.  in: channels-last activations; weights: [G][K][Ci][Co];
/// bias may be null; fp32 accumulation.
hipError_t launchGeneric(const GenericDesc &d, int inType, int outType,
                         const void *in, const void *weights, const void *bias,
                         void *out, const QuarterInfo &q, hipStream_t stream);

/// dst[i0][i1][i2][i3] = src[...] where dst dimension j walks source dimension
/// perm[j]; srcDims are the source extents; elemBytes 1, 2 or 4.
hipError_t launchPermute4(const void *src, void *dst, const uint64_t srcDims[4],
                          const int perm[4], int elemBytes, hipStream_t stream);

/// dst[g * strideG + c * strideC + p * strideP + b] = src[b][p][g][c]
/// (strides in elements; elements of 2 or 4 bytes): channels-last activations
/// with the batch axis moved innermost, as the weight update pass wants both
/// of its operands.
/// Weights in external order [groups][co][ci][taps] -> the block-diagonal
/// weights [groups / perGroup][perGroup co][perGroup ci][taps] of the layer
/// with `perGroup` neighbouring groups taken as one.
hipError_t launchFuseGroupWeights(const void *src, void *dst, uint64_t groups,
                                  uint64_t perGroup, uint64_t co, uint64_t ci,
                                  uint64_t taps, int elemBytes,
                                  hipStream_t stream);
/// ... and back, for weight deltas: the diagonal blocks of
/// [groups / perGroup][perGroup co][perGroup ci][taps] -> [groups][co][ci][taps].
hipError_t launchUnfuseGroupWeights(const void *src, void *dst,
                                    uint64_t groups, uint64_t perGroup,
                                    uint64_t co, uint64_t ci, uint64_t taps,
                                    int elemBytes, hipStream_t stream);
hipError_t launchSwapBatchChans(const void *src, void *dst, uint32_t batch,
                                uint32_t pixels, uint32_t groups,
                                uint32_t chans, uint64_t strideG,
                                uint64_t strideC, uint64_t strideP,
                                int elemBytes, hipStream_t stream);
/// Two of them (same element size) in one launch where both take the vector
/// path; otherwise one after the other.
struct SwapBatchChans {
  const void *src;
  void *dst;
  uint32_t batch, pixels, groups, chans;
  uint64_t strideG, strideC, strideP;
};
hipError_t launchSwapBatchChansPair(const SwapBatchChans &first,
                                    const SwapBatchChans &second,
                                    int elemBytes, hipStream_t stream);

/// Zero-fills `bytes` (a multiple of 4) with a kernel, so that the call can
/// be recorded into a graph.
hipError_t launchZero(void *dst, uint64_t bytes, hipStream_t stream);
/// out[image][fullD][fullH][fullW][chans] (kHalf or kFloat): every element
/// outside planes [offD, offD + insideD) x rows [offH, offH + insideH) x
/// columns [offW, offW + insideW) becomes bias[channel], or 0 without a bias;
/// the inside is not touched.
hipError_t launchFillOutputPadding(int type, void *out, const void *bias,
                                   uint64_t images, uint32_t fullD,
                                   uint32_t fullH, uint32_t fullW,
                                   uint32_t offD, uint32_t offH,
                                   uint32_t offW, uint32_t insideD,
                                   uint32_t insideH, uint32_t insideW,
                                   uint32_t chans, hipStream_t stream);

/// biases[c] += scale * sum over rows of zDeltas[row][c] (half or float each),
/// summed in fp32 in a fixed order: per-split partial sums go to `workspace`
/// (biasUpdateWorkspaceBytes), a second kernel adds them up split by split.
size_t biasUpdateWorkspaceBytes(uint64_t rows, uint64_t channels);
hipError_t launchBiasUpdate(int deltasType, const void *zDeltas, uint64_t rows,
                            uint64_t channels, int biasType, void *biases,
                            float scale, void *workspace, hipStream_t stream);

/// a[i] = scaleA * a[i] + scaleB * b[i] for half or float arrays, evaluated
/// in fp32.
hipError_t launchScaledAdd(int type, void *a, float scaleA, const void *b,
                           float scaleB, uint64_t total, hipStream_t stream);

/// dst[g][ci][co][k...] = src[g][co][ci][flipped k...]: channels transposed,
/// every one of the numDims (<= kMaxDims) kernel axes reversed.
hipError_t launchWeightsTransposeChansFlipXY(const void *src, void *dst,
                                             uint64_t groups, uint64_t co,
                                             uint64_t ci, uint32_t numDims,
                                             const uint32_t *kernelShape,
                                             int elemBytes,
                                             hipStream_t stream);

/// [pixels][groups][ci] -> [pixels][groups][ciPadded], the new channels zero;
/// ciPadded * elemBytes is a multiple of 16.
hipError_t launchPadChans(const void *src, void *dst, uint64_t pixels,
                          uint32_t groups, uint32_t ci, uint32_t ciPadded,
                          int elemBytes, hipStream_t stream);

/// Weights [G][Co][Ci][taps] -> [G][coPadded][kPadded] with k = tap * Ci + ci,
/// zero-filled beyond Co and beyond taps * Ci: the B operand of the
/// matrix-core kernel, K contiguous.  With ciPadded (not 0) every tap takes
/// ciPadded places of k, the ones beyond Ci zero.
/// `select` (optional) packs a sub-kernel: of a kH x kW kernel the taps
/// (firstH + i * stepH, firstW + j * stepW), i < countH, j < countW, in that
/// order; `taps` is then kH * kW of the source and K holds countH * countW of
/// them (none: all zeros).
struct IgemmTapSelection {
  uint32_t kW;
  uint32_t firstH, stepH, countH, firstW, stepW, countW;
  // the same along a depth: planes firstD + a * stepD, a < countD, of a
  // kernel of kH rows per plane (1 plane, unselected, by default)
  uint32_t kH = 1, firstD = 0, stepD = 1, countD = 1;
};
hipError_t launchPackIgemmWeights(const void *src, void *dst, uint32_t groups,
                                  uint32_t co, uint32_t ci, uint32_t taps,
                                  uint32_t coPadded, uint32_t kPadded,
                                  int elemBytes, hipStream_t stream,
                                  bool chansTransposed = false,
                                  uint32_t ciPadded = 0,
                                  const IgemmTapSelection *select = nullptr);

/// acts[outer][c] += bias[c] for `type` elements (kHalf or kFloat).
hipError_t launchAddBias(int type, void *acts, const void *bias,
                         uint64_t outerElems, uint64_t channels,
                         hipStream_t stream);

/// Implicit-GEMM forward convolution on the matrix cores: float, half or
/// quarter operands; a field of up to three dimensions with stride, zero
/// padding, truncation and kernel dilation; a dilated (zero-stuffed) input in
/// two dimensions.
struct IgemmDesc {
  uint32_t batch, groups, inChansPerGroup, outChansPerGroup;
  uint32_t inH, inW, outH, outW, kH, kW;
  // input row = outRow * strideH + kRow * dilH - padH, read when it lies in
  // [loH, hiH) and taken as zero otherwise; the same along W.
  int32_t padH, padW;
  uint32_t strideH, strideW, dilH, dilW;
  uint32_t loH, hiH, loW, hiW;
  // Tile shape chosen by the planner.
  uint32_t blockM, blockN, blockK;
  // A third, outermost field dimension (depth), with the same meaning of its
  // members; 1 / 0 where a field has none.  Kernels of at most 32 taps on
  // undilated inputs only.
  uint32_t inD = 1, outD = 1, kD = 1;
  int32_t padD = 0;
  uint32_t strideD = 1, dilD = 1, loD = 0, hiD = 1;
  // Where the outputs go: pixel (oh, ow) of this convolution is pixel
  // (oh * outStepH + outOffH, ow * outStepW + outOffW) of an output tensor
  // with outFullH x outFullW pixels per image (0: the convolution's own
  // field).  That is how one phase of a convolution over a zero-stuffed input
  // - the outputs whose windows meet the same residue of real input rows and
  // columns - writes its share of the whole output.  The same along the
  // depth (outFullD 0: the convolution's own).
  uint32_t outFullH = 0, outFullW = 0;
  uint32_t outStepH = 1, outStepW = 1, outOffH = 0, outOffW = 0;
  uint32_t outFullD = 0, outStepD = 1, outOffD = 0;
  // No tap of the kernel ever reads real input (a phase of a zero-stuffed
  // input that only meets stuffed zeros): the outputs are the bias, or zero,
  // and the workgroups run no k-step at all.
  uint32_t noTaps = 0;
  // Write the result as [channel][pixel] instead of [pixel][channel]: a
  // weight update pass's result in weight order.  Element stores - for small
  // outputs.  Not together with the output mapping above.
  uint32_t outTransposed = 0;
  // Zeros stuffed between input elements: input row r sits at row r * inDilH
  // of the field the window slides over (padH, strideH, dilH are in those
  // coordinates; loH, hiH bound r itself).  1 = none.
  uint32_t inDilH = 1, inDilW = 1;
  // Parts K is cut into, one workgroup each; above 1 the launch needs
  // igemmWorkspaceBytes of scratch and adds the parts up in a second kernel.
  uint32_t splitK = 1;
  // LDS stages of the 128-wide tile: 4 (one workgroup per CU, deep prefetch)
  // or 2 (two workgroups per CU, which cover each other's start-up, barriers
  // and epilogue: for grids of more workgroups than CUs).  The 64-wide tile
  // always runs 3.
  uint32_t stages = 4;
  // 1 or 2: the kernel that keeps a tile's input patch in LDS runs (unit
  // stride, channels in whole 128-byte slices; igemmPatchTakes); the packed
  // weights then have its layout (launchPackIgemmPatchWeights).  1: 32-pixel
  // MFMA blocks, blockM 64 or 128; 2: 16-pixel MFMA blocks, blockM = pixels
  // per tile, any number up to 112.
  uint32_t patch = 0;
  // Patch rows the tallest tile of that kernel spans (igemmPatchMaxRows),
  // worked out once when the plan is made - it takes a walk over the tiles -
  // so that a launch does not repeat it; 0 = not known, work it out.
  uint32_t patchMaxRows = 0;
};
/// How the kernel finds out which kernel taps of an output pixel read inside
/// the input: a bit mask per pixel (up to 32 taps), ranges of valid kernel
/// rows and columns per pixel (more taps), or arithmetic per tap (dilated
/// input).
enum : int { kMaskTaps = 0, kRangeTaps = 1, kDilatedTaps = 2 };
/// Whether the kernel can address the input: it uses 32-bit offsets from the
/// first image (batch element) a tile of 128 output rows reads, so those few
/// images - not the tensor - have to stay under 2^31 bytes.
bool igemmAddressable(const IgemmDesc &d, int inType);
int igemmTapAddressing(const IgemmDesc &d);
size_t igemmWorkspaceBytes(const IgemmDesc &d);
hipError_t launchIgemm(const IgemmDesc &d, int inType, int outType,
                       const void *in, const void *weightsPacked,
                       const void *bias, void *out, void *workspace,
                       const QuarterInfo &q, hipStream_t stream);

/// The same convolution by the kernel that loads the input rows a tile reads
/// into LDS once and forms every tap's operand by LDS addressing: unit stride,
/// undilated input, two field dimensions, half or quarter inputs whose
/// channels per group fill whole 128-byte slices, K not split.
bool igemmPatchTakes(const IgemmDesc &d, int inType, int outType);
/// Patch rows a tile of d.blockM consecutive output pixels can span: what a
/// planner stores in d.patchMaxRows.
uint32_t igemmPatchMaxRows(const IgemmDesc &d);
/// Elements of its packed weights:
/// [G][32-channel block][K half][k-step][operand][lane][16 bytes].
uint64_t igemmPatchPackedElems(const IgemmDesc &d, int inType);
/// src as for launchPackIgemmWeights; sourceTaps: taps of the stored kernel.
hipError_t launchPackIgemmPatchWeights(const IgemmDesc &d, int inType,
                                       const void *src, void *dst,
                                       uint32_t sourceTaps, hipStream_t stream,
                                       bool chansTransposed = false,
                                       const IgemmTapSelection *select =
                                           nullptr);
hipError_t launchIgemmPatch(const IgemmDesc &d, int inType, int outType,
                            const void *in, const void *weightsPacked,
                            const void *bias, void *out, const QuarterInfo &q,
                            hipStream_t stream);

/// Several convolutions that run the same igemm kernel (same tile width,
/// types, fp8 formats, channel-block alignment; K not split) as ONE launch
/// whose grid is the concatenation of their tiles - at most 8 at a time.
struct IgemmFusedItem {
  const IgemmDesc *d;
  int inType, outType;
  const void *in, *weightsPacked, *bias;
  void *out;
  QuarterInfo q;
};
constexpr size_t kIgemmMaxFused = 8;
bool igemmFusable(const IgemmFusedItem &x, const IgemmFusedItem &y);
hipError_t launchIgemmFused(const IgemmFusedItem *items, size_t count,
                            hipStream_t stream);

/// Pointwise convolution (every kernel extent 1, stride 1, no padding or
/// truncation, half inputs) with a multiple of 8 up to 512 input channels per
/// group: a streaming kernel of small workgroups instead of igemm's big tiles
/// (compiled for rows of 16, 32, 64, 128, 256 and 512 channels; a layer in
/// between runs as the next one up).
struct PointwiseDesc {
  uint32_t batch, pixels; // pixels per image
  uint32_t groups, inChansPerGroup, outChansPerGroup;
  // 64-channel tiles of the output a workgroup owns: 0 = the launch's choice
  uint32_t chanTiles = 0;
  // bytes of an input element: 2 (fp16) or 1 (fp8)
  uint32_t elemBytes = 2;
};
bool pointwiseTakes(const PointwiseDesc &d, int inType, int outType);
/// Whether a workgroup can own `chanTiles` 64-channel tiles of this layer's
/// output (they divide the layer's; 4 at most with 64 input channels, 2 with
/// 128 or 256, 1 with 512).
bool pointwiseChanTilesOk(const PointwiseDesc &d, uint32_t chanTiles);
/// Elements of the packed weights ([G][32-channel block][32-byte k-slice]
/// [lane][16 bytes]).
uint64_t pointwisePackedElems(const PointwiseDesc &d);
hipError_t launchPackPointwiseWeights(const PointwiseDesc &d, const void *src,
                                      void *dst, hipStream_t stream,
                                      bool chansTransposed = false);
/// How launchPointwise runs a layer on a chip of `cus` compute units:
/// persistent workgroups, each taking tiles of `tilePixels` pixels in turn
/// through a ring of `ring` LDS buffers filled by `loaderWaves` waves.
struct PointwiseLaunch {
  uint32_t tilePixels, ring, loaderWaves, tilesPerWorkgroup;
  uint32_t chansPerWorkgroup; // 64, 128 or 256 output channels
  uint64_t workgroups;
};
PointwiseLaunch pointwiseLaunchShape(const PointwiseDesc &d, uint32_t cus);
hipError_t launchPointwise(const PointwiseDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, const QuarterInfo &q,
                           hipStream_t stream);

/// Convolution of an input with 1 to 4 channels (one group, half inputs, a
/// 2-D field, stride, zero padding, input truncation; nothing dilated) on the
/// matrix cores without padding the channels: a kernel row's kW * Ci
/// neighbouring elements (32 at most), in chunks of 8, fill k-steps of 32.
/// 16, 32, 48 or 64 output channels, up to 28 chunks (7 k-steps).
struct ThinInputDesc {
  uint32_t batch, inChans, outChans;
  uint32_t inH, inW, outH, outW, kH, kW;
  int32_t padH, padW; // as in IgemmDesc; padW >= 0
  uint32_t strideH, strideW;
  uint32_t loH, hiH, loW, hiW; // rows and columns outside read as zeros
};
bool thinInputTakes(const ThinInputDesc &d, int inType, int outType);
/// Elements of the packed weights ([16-channel block][k-step][lane][8]).
uint64_t thinInputPackedElems(const ThinInputDesc &d);
/// k-steps of 32: a kernel row is ceil(kW * Ci / 8) chunks of 8 elements,
/// four chunks make a k-step.
uint32_t thinInputKSteps(const ThinInputDesc &d);
hipError_t launchPackThinInputWeights(const ThinInputDesc &d, const void *src,
                                      void *dst, hipStream_t stream);
/// How launchThinInput runs a layer on a chip of `cus` compute units:
/// persistent workgroups, each taking tiles of `tileRows` output rows of one
/// image in turn, the input rows under a tile in `ldsBytes` of LDS.
struct ThinInputLaunch {
  uint32_t tileRows, ldsBytes;
  uint64_t tiles, workgroups;
};
ThinInputLaunch thinInputLaunchShape(const ThinInputDesc &d, uint32_t cus);
hipError_t launchThinInput(const ThinInputDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, hipStream_t stream);

/// Depthwise (one input and one output channel per group) direct convolution,
/// 2-D field, stride, zero padding, kernel dilation.
struct DepthwiseDesc {
  uint32_t batch, channels;
  uint32_t inH, inW, outH, outW, kH, kW;
  int32_t padH, padW; // as in IgemmDesc
  uint32_t strideH, strideW, dilH, dilW;
  uint32_t loH, hiH, loW, hiW;
  // Output pixels per workgroup tile, chosen by the planner so that the
  // input patch of a tile fits a third of a CU's LDS.
  uint32_t tileH, tileW;
  // 3x3 taps, dilation 1, stride 1 or 2 - 1: the dense-loading
  // small-workgroup kernel, 2: the persistent kernel with a ring of input rows
  // in LDS (launchDepthwiseRows), instead of the LDS-tiled one.
  uint32_t dense3x3;
  // Compute units the persistent kernel spreads its workgroups over.
  uint32_t cus = 0;
  // Zeros stuffed between input elements, as in IgemmDesc; other than 1 the
  // direct kernel of launchDepthwiseDirect runs.
  uint32_t inDilH = 1, inDilW = 1;
  // The LDS-tiled kernel with a thread forming that many neighbouring output
  // pixels of a row at once (7 x 7 taps, unit stride and dilation:
  // depthwiseStripTakes): 4 or 7; 0 = a pixel at a time.
  uint32_t stripPixels = 0;
  // Bytes of an input element: 2 (fp16: every depthwise kernel), 4 (fp32) or
  // 1 (fp8) - those two by the LDS-tiled kernel only.
  uint32_t elemBytes = 2;
};
/// True for the layers whose LDS-tiled kernel can work in strips of pixels.
bool depthwiseStripTakes(const DepthwiseDesc &d);
/// LDS of a workgroup of the LDS-tiled kernel for d's tile: the input patch
/// and, with strips, the taps; what it may take at most.
uint64_t depthwiseTileLdsBytes(const DepthwiseDesc &d);
constexpr uint32_t kDepthwiseTileLdsMost = 80 * 1024;
/// True for the shapes launchDepthwise3x3 takes.
bool depthwise3x3Takes(const DepthwiseDesc &d, int inType);
hipError_t launchDepthwise3x3(const DepthwiseDesc &d, int inType,
                                 int outType, const void *in,
                                 const void *weightsPacked, const void *bias,
                                 void *out, hipStream_t stream);
/// The same layers (3x3 taps, dilation 1, stride 1 or 2) by persistent
/// workgroups, about one per compute unit (d.cus), each walking down a band
/// of output rows of a column strip with the input rows in an LDS ring.
bool depthwiseRowsTakes(const DepthwiseDesc &d, int inType);
struct DepthwiseRowsLaunch {
  uint32_t strips, colsOut, bands, rowsOut, ringRows, loaderWaves;
  uint32_t computeWaves;
  uint64_t workgroups;
};
DepthwiseRowsLaunch depthwiseRowsLaunchShape(const DepthwiseDesc &d);
hipError_t launchDepthwiseRows(const DepthwiseDesc &d, int inType, int outType,
                               const void *in, const void *weightsPacked,
                               const void *bias, void *out,
                               hipStream_t stream);
/// The weight deltas of such a layer the same way: one fp32 tile [9][C] per
/// workgroup at partial[workgroup], to be added in order; *walkers = their
/// count.
bool depthwiseRowsDeltaTakes(const DepthwiseDesc &d);
DepthwiseRowsLaunch depthwiseRowsDeltaLaunchShape(const DepthwiseDesc &d);
size_t depthwiseRowsDeltaWorkspaceBytes(const DepthwiseDesc &d);
hipError_t launchDepthwiseRowsDeltas(const DepthwiseDesc &d, const void *acts,
                                     const void *deltas, void *partial,
                                     uint32_t *walkers, hipStream_t stream);
hipError_t launchDepthwise(const DepthwiseDesc &d, int inType, int outType,
                           const void *in, const void *weightsPacked,
                           const void *bias, void *out, const QuarterInfo &q,
                           hipStream_t stream);
/// The same convolution by one thread per output vector, reading the input
/// from global memory; takes a dilated input (d.inDilH, d.inDilW), ignores
/// the tile fields.
hipError_t launchDepthwiseDirect(const DepthwiseDesc &d, int inType,
                                 int outType, const void *in,
                                 const void *weightsPacked, const void *bias,
                                 void *out, hipStream_t stream);
/// True when launchDepthwiseDirect serves `d` with its kernel of one thread
/// per block of outputs (input dilated by 2 in both dimensions, unit stride
/// and kernel dilation, 3x3 or 5x5 taps: the backward pass of a stride-2
/// layer), which loads every input vector and tap once per thread.
bool depthwiseDirectInBlocks(const DepthwiseDesc &d);
/// The FORWARD convolution of a dense layer whose weight deltas
/// launchWuTap forms from the layer's own tensors: two field dimensions, unit
/// stride, nothing dilated, truncated or flipped, fp16 tensors, channels in
/// whole 16-byte vectors.  An input pixel of output (y, x) and tap (kh, kw) is
/// (y + kh - padH, x + kw - padW), read when it lies in [loH, hiH) x
/// [loW, hiW), else zero.
struct WuTapDesc {
  uint32_t batch, inH, inW, outH, outW, kH, kW;
  int32_t padH, padW;
  uint32_t loH, hiH, loW, hiW;
  uint32_t groups, ci, co;
  // pixels (batch, y, x flattened) a workgroup sums over: a multiple of 64
  uint32_t chunkPixels;
  // the layer's stride: output pixel (y, x) meets input pixel
  // (y strideH + kh - padH, x strideW + kw - padW)
  uint32_t strideH = 1, strideW = 1;
};
bool wuTapTakes(const WuTapDesc &d);
/// Pixels per workgroup that give about one workgroup per compute unit.
uint32_t wuTapChunkPixels(const WuTapDesc &d, uint32_t computeUnits);
uint64_t wuTapWorkspaceBytes(const WuTapDesc &d);
/// weightDeltas [groups][co][ci][kH][kW] in outType (half or float) from acts
/// [batch][inH][inW][groups][ci] and deltas [batch][outH][outW][groups][co],
/// both fp16; fp32 partial tiles of the pixel chunks go through `workspace`
/// and are added in a fixed order.
hipError_t launchWuTap(const WuTapDesc &d, int outType, const void *acts,
                       const void *deltas, void *workspace, void *out,
                       hipStream_t stream);

/// Gradient with respect to the weights of the depthwise FORWARD convolution
/// `d` (undilated input): weightDeltas [channels][kH * kW] in outType from
/// acts [batch][inH][inW][channels] and deltas [batch][outH][outW][channels],
/// both fp16.  Partial sums over slices of the pixels go through `workspace`
/// and are added in a fixed order.
size_t depthwiseWeightDeltaWorkspaceBytes(const DepthwiseDesc &d);
hipError_t launchDepthwiseWeightDeltas(const DepthwiseDesc &d, int outType,
                                       const void *acts, const void *deltas,
                                       void *workspace, void *weightDeltas,
                                       hipStream_t stream);

} // namespace mxk
#endif

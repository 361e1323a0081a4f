#include "Plan.hpp"
#include "poplar/exceptions.hpp"
#include "poplin/ConvUtil.hpp"
#include "poputil/exceptions.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <sstream>
#include <vector>

namespace poplin {

namespace {

std::size_t product(const std::vector<std::size_t> &v) {
  std::size_t p = 1;
  for (auto x : v)
    p *= x;
  return p;
}

mxk::DimTransform toDim(const std::vector<std::size_t> &shape,
                        const ConvParams::InputTransform &t, unsigned d,
                        unsigned transformedSize) {
  return {uint32_t(shape[d]), t.truncationLower[d], t.truncationUpper[d],
          t.dilation[d],      t.paddingLower[d],    t.paddingUpper[d],
          uint32_t(t.flip[d] ? 1 : 0), transformedSize};
}

mxk::GenericDesc makeGenericDesc(const ConvParams &p) {
  mxk::GenericDesc g{};
  g.numDims = uint32_t(p.getNumFieldDims());
  g.batch = uint32_t(p.batchSize);
  g.groups = uint32_t(p.numConvGroups);
  g.inChansPerGroup = uint32_t(p.inputChannelsPerConvGroup);
  g.outChansPerGroup = uint32_t(p.outputChannelsPerConvGroup);
  g.kernelElems = 1;
  g.outElems = uint64_t(p.batchSize) * p.getNumOutputChans();
  for (unsigned d = 0; d != g.numDims; ++d) {
    g.in[d] = toDim(p.inputFieldShape, p.inputTransform, d,
                    p.getTransformedInputSize(d));
    g.kernel[d] = toDim(p.kernelShape, p.kernelTransform, d,
                        p.getTransformedKernelSize(d));
    g.outSize[d] = uint32_t(p.getOutputSize(d));
    g.outTruncLo[d] = p.outputTransform.truncationLower[d];
    g.outStride[d] = p.outputTransform.stride[d];
    g.outPadLo[d] = p.outputTransform.paddingLower[d];
    g.outPadHi[d] = p.outputTransform.paddingUpper[d];
    g.kernelElems *= uint32_t(p.kernelShape[d]);
    g.outElems *= g.outSize[d];
  }
  return g;
}

/// The subset the fast kernels take: up to two field dimensions; input with
/// truncation, dilation and zero padding; kernel with dilation only; output
/// with truncation and stride only.  Written as "row of the dilated input =
/// out*stride + k*dilation - pad; it holds input row r when it equals
/// r*inDil, valid for r inside [lo, hi)".
struct Simple2D {
  bool ok = false;
  std::string why;
  uint32_t inH = 1, inW = 1, outH = 1, outW = 1, kH = 1, kW = 1;
  int32_t padH = 0, padW = 0;
  uint32_t strideH = 1, strideW = 1, dilH = 1, dilW = 1;
  uint32_t loH = 0, hiH = 1, loW = 0, hiW = 1;
  uint32_t inDilH = 1, inDilW = 1;
  // A third, outermost dimension (depth).  One that the window does not
  // slide over in any interesting way (kernel 1, stride 1, nothing padded,
  // truncated or dilated) is folded into the batch instead.
  uint32_t inD = 1, outD = 1, kD = 1;
  int32_t padD = 0;
  uint32_t strideD = 1, dilD = 1, loD = 0, hiD = 1, inDilD = 1;
  std::size_t batch = 0; // the batch size times the folded depth
  // Kernel truncation, padding and flips: the kernel the window applies
  // (kD, kH, kW) is a selection of the taps of the stored one - tap j of it
  // is stored tap first + j * step (step 1, or -1 for a flipped dimension) -
  // and kernel padding only moves the window (folded into pad).  fullK*: the
  // stored extents.
  bool kernelSelected = false;
  uint32_t fullKD = 1, fullKH = 1, fullKW = 1;
  uint32_t selFirstD = 0, selFirstH = 0, selFirstW = 0;
  uint32_t selStepD = 1, selStepH = 1, selStepW = 1; // 1 or uint32_t(-1)
  // Zeros around the output field (outH, outW are the convolution's own).
  uint32_t outPadLoH = 0, outPadHiH = 0, outPadLoW = 0, outPadHiW = 0;
  uint32_t outPadLoD = 0, outPadHiD = 0;
  bool outputPadded() const {
    return outPadLoH || outPadHiH || outPadLoW || outPadHiW || outPadLoD ||
           outPadHiD;
  }
  bool hasDepth() const { return inD != 1 || outD != 1 || kD != 1; }
  bool inputDilated() const {
    return inDilH != 1 || inDilW != 1 || inDilD != 1;
  }
};

Simple2D asSimple2D(const ConvParams &p) {
  Simple2D s;
  const unsigned n = unsigned(p.getNumFieldDims());
  if (n > 3) {
    s.why = "more than three field dimensions";
    return s;
  }
  s.batch = p.batchSize;
  for (unsigned d = 0; d != n; ++d) {
    const auto &it = p.inputTransform, &kt = p.kernelTransform;
    const auto &ot = p.outputTransform;
    if (it.flip[d]) {
      s.why = "input flip";
      return s;
    }
    const bool kernelTransformed =
        kt.truncationLower[d] || kt.truncationUpper[d] || kt.paddingLower[d] ||
        kt.paddingUpper[d] || kt.flip[d];
    if (kt.truncationLower[d] + kt.truncationUpper[d] >= p.kernelShape[d] &&
        kernelTransformed) {
      s.why = "kernel truncated to nothing";
      return s;
    }
    // conv index = o*stride + outTruncLo; padded input = conv + k*dil;
    // dilated input = padded - padLo; input = dilated / inDil + truncLo when
    // that is whole.
    // (kernel padding shifts where the taps sit in the window: the lower
    // one, or - the flip comes last - the upper one of a flipped kernel)
    const int32_t pad =
        int32_t(it.paddingLower[d]) -
        int32_t(it.truncationLower[d] * it.dilation[d]) -
        int32_t(ot.truncationLower[d]) -
        int32_t(kt.flip[d] ? kt.paddingUpper[d] : kt.paddingLower[d]);
    const uint32_t kept = uint32_t(p.kernelShape[d] - kt.truncationLower[d] -
                                   kt.truncationUpper[d]);
    const uint32_t lo = it.truncationLower[d];
    const uint32_t hi = uint32_t(p.inputFieldShape[d]) - it.truncationUpper[d];
    // which of depth, height, width: the innermost dimension is the width
    const unsigned which = d + 3 - n;
    auto pick = [which](auto &dd, auto &hh, auto &ww) -> auto & {
      return which == 0 ? dd : which == 1 ? hh : ww;
    };
    pick(s.inD, s.inH, s.inW) = uint32_t(p.inputFieldShape[d]);
    pick(s.outD, s.outH, s.outW) = uint32_t(
        p.getOutputSize(d) - ot.paddingLower[d] - ot.paddingUpper[d]);
    pick(s.outPadLoD, s.outPadLoH, s.outPadLoW) = ot.paddingLower[d];
    pick(s.outPadHiD, s.outPadHiH, s.outPadHiW) = ot.paddingUpper[d];
    pick(s.kD, s.kH, s.kW) = kept;
    pick(s.fullKD, s.fullKH, s.fullKW) = uint32_t(p.kernelShape[d]);
    pick(s.selFirstD, s.selFirstH, s.selFirstW) =
        kt.flip[d] ? uint32_t(kt.truncationLower[d]) + kept - 1
                   : uint32_t(kt.truncationLower[d]);
    pick(s.selStepD, s.selStepH, s.selStepW) = kt.flip[d] ? ~0u : 1u;
    s.kernelSelected = s.kernelSelected || kernelTransformed;
    pick(s.padD, s.padH, s.padW) = pad;
    pick(s.strideD, s.strideH, s.strideW) = ot.stride[d];
    pick(s.dilD, s.dilH, s.dilW) = kt.dilation[d];
    pick(s.loD, s.loH, s.loW) = lo;
    pick(s.hiD, s.hiH, s.hiW) = hi;
    pick(s.inDilD, s.inDilH, s.inDilW) = it.dilation[d];
  }
  if (s.kD == 1 && s.strideD == 1 && s.padD == 0 && s.loD == 0 &&
      s.hiD == s.inD && s.inDilD == 1 && s.outD == s.inD &&
      s.outPadLoD == 0 && s.outPadHiD == 0) {
    s.batch *= s.inD;
    s.inD = s.outD = s.hiD = 1;
  }
  s.ok = true;
  return s;
}

/// Output tile (height, width) of the depthwise kernel: the input patch of a
/// tile - ((th-1)*stride + (k-1)*dilation + 1 rows, likewise columns, for up
/// to 16 channel vectors of 16 bytes - has to fit 52 KB so that three
/// workgroups share the 160 KB of a CU.  Width first: the candidate (at most
/// 16) that wastes the fewest pixels at the right edge; then the tallest tile
/// that fits.  {0, 0} when not even one pixel fits.
std::pair<unsigned, unsigned> chooseDepthwiseTile(const Simple2D &s,
                                                  std::size_t vecs) {
  const std::size_t vecBlock = std::min<std::size_t>(vecs, 16);
  const std::size_t budget = (52 * 1024) / 16; // 16-byte elements
  auto patch = [](unsigned t, unsigned stride, unsigned k, unsigned dil) {
    return std::size_t(t - 1) * stride + std::size_t(k - 1) * dil + 1;
  };
  for (unsigned maxW = 16; maxW >= 1; maxW /= 2) {
    unsigned bestW = 0;
    std::size_t bestWaste = ~std::size_t(0);
    for (unsigned tw = std::min(maxW, s.outW); tw > maxW / 2; --tw) {
      const std::size_t waste = (s.outW + tw - 1) / tw * tw - s.outW;
      if (waste < bestWaste) {
        bestWaste = waste;
        bestW = tw;
      }
    }
    if (bestW == 0)
      continue;
    const std::size_t pw = patch(bestW, s.strideW, s.kW, s.dilW);
    unsigned bestH = 0;
    for (unsigned th = 1; th <= std::min(16u, s.outH); ++th)
      if (patch(th, s.strideH, s.kH, s.dilH) *
              ((pw * vecBlock + 63) / 64 * 64) <=
          budget) // rows are padded to whole 64-element loads
        bestH = th;
    if (bestH)
      return {bestH, bestW};
  }
  return {0, 0};
}

/// Tile and strip of the LDS-tiled depthwise kernel where a thread forms a
/// strip of neighbouring pixels (mxk::depthwiseStripTakes): such layers cost
/// what their multiply-adds cost, so the tile is the one that keeps most of a
/// workgroup's 256 threads busy - rows x strips x channel vectors close to a
/// multiple of 256, few rows beyond the field's last, strips of seven pixels
/// where the tile's width is a multiple of seven and of four elsewhere
/// (ConvNeXt's 7 x 7 field: two strips of four, 224 threads, against one of
/// seven, 112) - within the LDS two workgroups of a CU can have.
/// Busy share of a workgroup's threads with strips of `px` pixels on a tile.
double stripFill(const mxk::DepthwiseDesc &d, unsigned th, unsigned tw,
                 unsigned px) {
  const unsigned vb = std::min(d.channels / 8, 16u);
  const unsigned strips = (tw + px - 1) / px;
  const double lanes = double(th) * strips * vb;
  return lanes / (std::ceil(lanes / 256.0) * 256.0) * double(tw) /
         (strips * px);
}

/// Strips of seven pixels where the tile's width is a multiple of seven and
/// that keeps at least as many threads busy as strips of four.
unsigned stripPixelsFor(const mxk::DepthwiseDesc &d, unsigned th,
                        unsigned tw) {
  return tw % 7 == 0 && stripFill(d, th, tw, 7) >= stripFill(d, th, tw, 4)
             ? 7
             : 4;
}

void chooseDepthwiseStripTile(mxk::DepthwiseDesc &d) {
  const unsigned vecs = d.channels / 8, vb = std::min(vecs, 16u);
  // (channel blocks of 16 vectors: the last block's share of busy lanes)
  const double chanFill =
      double(vecs) / double((vecs + vb - 1) / vb * vb);
  double best = 0;
  mxk::DepthwiseDesc chosen = d;
  for (unsigned tw = 1; tw <= std::min(16u, d.outW); ++tw)
    for (unsigned th = 1; th <= std::min(32u, d.outH); ++th) {
      mxk::DepthwiseDesc t = d;
      t.tileH = th, t.tileW = tw, t.stripPixels = stripPixelsFor(d, th, tw);
      if (mxk::depthwiseTileLdsBytes(t) > mxk::kDepthwiseTileLdsMost)
        break;
      const double edgeH =
          double(d.outH) / double((d.outH + th - 1) / th * th);
      const double edgeW =
          double(d.outW) / double((d.outW + tw - 1) / tw * tw);
      // (the patch's halo is loaded, not multiplied: a quarter's weight)
      const double halo = double(th) * tw / (double(th + 6) * (tw + 6));
      const double score = stripFill(d, th, tw, t.stripPixels) * edgeH *
                           edgeW * chanFill * (0.75 + 0.25 * halo);
      if (score > best)
        best = score, chosen = t;
    }
  d = chosen;
}

} // namespace

namespace {

// Cost model of the matrix-core kernels, in microseconds, from kernel traces
// and in-kernel cycle stamps on MI355X at the ~2.0 GHz the chip holds under
// MFMA load.  A k-step is 128 bytes of K per tile row.
constexpr double kLaunchUs = 2.0; // dispatch + drain of any kernel

/// Rounds of workgroups a launch makes with `perCU` workgroups per CU: whole
/// ones where one workgroup owns a CU (equal tiles all end together), softer
/// where two share it.
double roundsOf(std::size_t workgroups, std::size_t perCU) {
  const double slots = double(gfx950::numCUs) * double(perCU);
  if (double(workgroups) <= slots)
    return 1.0;
  const double whole = std::ceil(double(workgroups) / slots);
  return perCU == 1 ? whole : std::min(whole, double(workgroups) / slots + 0.5);
}

/// igemmKernel: 1.45 us start-up + 1.5 us epilogue, 0.345 us per k-step of a
/// 128 x 128 tile (0.24 for 128 x 64); further rounds on a CU pay another
/// 1.5 us (nothing overlaps the next workgroup's start-up); two workgroups
/// sharing a CU take 2.1 times one's time between them; K split adds
/// splitPenaltyUs of its `partialBytes` of fp32 tiles.
/// What K split over workgroups adds: the second kernel with its launch, and
/// the fp32 partial tiles' way out and in again at what a stream of that size
/// reaches (N = 32, 14 x 14, 1 x 1, 1024 -> 256 in two parts, 12.8 MB of
/// tiles: 16.4 us where the tiles' k-steps are estimated at 7.7; 7 x 7, 3 x 3,
/// 512 -> 512 in four, 12.8 MB: 18.7 against 11.2; N = 1, 14 x 14, 3 x 3,
/// 256 -> 256 in nine, 1.8 MB: 9.2 against 6.3).
double splitPenaltyUs(std::size_t partialBytes) {
  return 4.5 + 2.0 * double(partialBytes) / 6.4e6;
}

double estimateStreaming(std::size_t workgroups, std::size_t kSteps,
                         std::size_t perCU, unsigned blockN, unsigned splitK,
                         std::size_t partialBytes) {
  const double rounds = roundsOf(workgroups, perCU);
  const double step = blockN == 128 ? 0.345 : 0.24;
  double tile = 2.95 + step * double(kSteps);
  if (perCU == 1 && rounds > 1)
    tile += 1.5;
  if (perCU == 2)
    tile *= double(workgroups) > double(gfx950::numCUs) ? 2.1 : 1.0;
  return kLaunchUs + rounds * tile +
         (splitK > 1 ? splitPenaltyUs(partialBytes) : 0.0);
}

/// igemmPatchKernel (mode 1): 1.9 us to the first MFMA + 0.5 us reduction and
/// stores, 0.333 us per k-step of 128 pixels (half of that for 64); one
/// workgroup per CU, so further rounds pay their start-up in full (4.5 us
/// instead of 2.4).  igemmPatch16Kernel (mode 2): seven blocks of 16 pixels
/// whatever the tile's height, 0.29 us per k-step and 1.5 us around them in
/// a launch of one round (8.6 us measured for 224 tiles of 18 k-steps, 17.1
/// for 50 k-steps), 0.34 and 2.6 us in launches of several (55 us for 4
/// rounds of 36, 110 us for 7 rounds of 36, 35 us for 4 rounds of 18).
double estimatePatch(std::size_t workgroups, std::size_t kSteps, unsigned mode,
                     unsigned blockM) {
  const double rounds = roundsOf(workgroups, 1);
  if (mode == 2)
    return kLaunchUs + rounds * ((rounds > 1 ? 2.6 : 1.5) +
                                 (rounds > 1 ? 0.34 : 0.29) * double(kSteps));
  const double step = blockM == 128 ? 0.333 : 0.167;
  const double fixed = rounds > 1 ? 4.5 : 2.4;
  return kLaunchUs + rounds * (fixed + step * double(kSteps));
}

} // namespace

namespace {

/// Conv groups to run as one (see mxconv_plan::convGroupsPerGroup), 1 = each
/// by itself.  By the planner's own choice: layers whose groups have fewer
/// input channels than half a 128-byte slice and few output channels - the
/// smallest number of groups that makes a whole slice, where that keeps the
/// fused group within 256 output channels (32 groups of 4 -> 4 channels run
/// as 2 groups of 64 -> 64: 16 times the multiply-adds, on matrix cores that
/// stood idle behind 16-byte vectors half empty and 64-channel tiles with 4
/// channels in them).  A `convGroupsPerGroup` plan constraint is taken where
/// it can be (it divides the groups and the fused channels are whole 16-byte
/// vectors) and means "by itself" elsewhere: the reference accepts values
/// that only its own vertices give a meaning to.
///
/// A weight update pass (its parameters are getWeightUpdateParams of the
/// layer's: batch = the layer's input channels, input channels = its batch)
/// is planned for the layer with that many groups taken as one - the same
/// rule on the layer's channels - and the diagonal blocks of the fused
/// layer's weight deltas are what the pass hands back
/// (mxconv_plan::wuGroupsPerGroup).
unsigned chooseConvGroupsPerGroup(const ConvParams &p,
                                  const ConvOptions &options) {
  const auto &pc = options.planConstraints;
  const bool wu = isWeightUpdatePass(options.pass);
  switch (options.pass) {
  case Pass::NONE:
  case Pass::INFERENCE_FWD:
  case Pass::TRAINING_FWD:
  case Pass::TRAINING_BWD:
  case Pass::TRAINING_WU:
    break;
  default:
    return 1;
  }
  const std::size_t groups = p.numConvGroups;
  const std::size_t ci = wu ? p.batchSize : p.inputChannelsPerConvGroup;
  const std::size_t co = p.outputChannelsPerConvGroup;
  const std::size_t eb = p.inputType.size();
  if (groups < 2 || ci == 0 || co == 0 || (ci == 1 && co == 1) ||
      (!pc.kernel.empty() && pc.kernel != "igemm") || p.batchSize == 0 ||
      p.inputChannelsPerConvGroup == 0)
    return 1;
  auto usable = [&](std::size_t f) {
    return f >= 1 && groups % f == 0 && (f * ci * eb) % 16 == 0;
  };
  if (pc.convGroupsPerGroup != 0)
    return usable(pc.convGroupsPerGroup) ? pc.convGroupsPerGroup : 1u;
  // (one input channel per group with several output channels - a depthwise
  // layer with a channel multiplier - included: 64 groups of 1 -> 2 channels
  // run as one of 64 -> 128)
  if (ci * eb >= 64)
    return 1;
  for (std::size_t f = 2; f <= groups; ++f)
    if (usable(f) && f * ci * eb >= 128)
      return f * co <= 256 ? unsigned(f) : 1u;
  // (too few groups for a whole slice: all of them, where that makes two
  // vectors of channels or more)
  if (usable(groups) && groups * ci * eb >= 32 && groups * co <= 256)
    return unsigned(groups);
  return 1;
}

mxconv_plan makePlanWith(const ConvParams &params,
                         const ConvOptions &optionsIn,
                         unsigned convGroupsPerGroup);

} // namespace

mxconv_plan makePlan(const ConvParams &params, const ConvOptions &optionsIn) {
  const unsigned fuse =
      chooseConvGroupsPerGroup(params.canonicalize(), optionsIn);
  if (fuse > 1 && isWeightUpdatePass(optionsIn.pass)) {
    // the weight update pass of the layer with `fuse` groups taken as one
    ConvParams fused = params;
    fused.numConvGroups /= fuse;
    fused.batchSize *= fuse;
    fused.outputChannelsPerConvGroup *= fuse;
    mxconv_plan plan = makePlanWith(fused, optionsIn, 1);
    plan.wuGroupsPerGroup = fuse;
    return plan;
  }
  if (fuse > 1) {
    // (only the matrix-core kernels run groups as one)
    mxconv_plan plan = makePlanWith(params, optionsIn, fuse);
    if (plan.kernel == mxconv_plan::Kernel::IGEMM)
      return plan;
  }
  return makePlanWith(params, optionsIn, 1);
}

namespace {

mxconv_plan makePlanWith(const ConvParams &params,
                         const ConvOptions &optionsIn,
                         unsigned convGroupsPerGroup) {
  mxconv_plan plan;
  plan.params = params;
  plan.canonical = params.canonicalize(); // validates
  plan.options = optionsIn;
  ConvOptions &options = plan.options;
  // What the kernels are planned for: the canonical parameters, with
  // `convGroupsPerGroup` groups taken as one further down.
  ConvParams planned = plan.canonical;
  const ConvParams &p = planned;

  if (p.getNumFieldDims() > mxk::kMaxDims)
    throw poputil::poplibs_error("At most " + std::to_string(mxk::kMaxDims) +
                                 " field dimensions are supported");

  // validateLayerParams: partials at least as wide as the output; quarter
  // inputs produce half outputs.  This build always accumulates in fp32, which
  // satisfies every partials type the reference would settle on.
  for (poplar::Type *t : {&options.partialsType, &options.interTilePartialsType,
                          &options.interIpuPartialsType})
    if (t->size() < params.outputType.size())
      *t = params.outputType;
  if (params.inputType == poplar::QUARTER && params.outputType != poplar::HALF)
    throw poputil::poplibs_error(
        "When the input type for a convolution is quarter, the output type "
        "must be half, not " +
        params.outputType.toString());
  if (params.outputType == poplar::QUARTER)
    throw poputil::poplibs_error("Unsupported convolution output element type "
                                 "(must be float or half)");

  plan.inputElems = params.batchSize * params.getNumInputChans() *
                    product(params.inputFieldShape);
  plan.outputElems = params.batchSize * params.getNumOutputChans() *
                     product(params.getOutputFieldShape());
  plan.weightElems = params.numConvGroups * params.outputChannelsPerConvGroup *
                     params.inputChannelsPerConvGroup *
                     product(params.kernelShape);
  plan.biasElems = params.getNumOutputChans();
  plan.generic = makeGenericDesc(p);
  plan.zeroConv = isZeroConvolution(p);
  plan.madeForWeightUpdate = isWeightUpdatePass(options.pass);

  using Kernel = mxconv_plan::Kernel;
  using Method = PlanConstraints::Method;
  // The weight update pass of a depthwise layer (getWeightUpdateParams of
  // it): one "image" (the layer's single input channel per group), one output
  // channel per group, the layer's batch as input channels.  Its output field
  // is the layer's kernel, its kernel the layer's output field, its kernel
  // dilation the layer's stride and its stride the layer's kernel dilation.
  {
    const Simple2D w = asSimple2D(p);
    if (isWeightUpdatePass(options.pass) &&
        options.planConstraints.weightDeltas != 0 && w.ok && !w.hasDepth() &&
        !w.outputPadded() && !w.kernelSelected && w.batch == 1 &&
        !plan.zeroConv &&
        !w.inputDilated() && p.batchSize == 1 &&
        p.outputChannelsPerConvGroup == 1 &&
        (params.inputType == poplar::HALF ||
         params.inputType == poplar::FLOAT) &&
        p.numConvGroups % (16 / params.inputType.size()) == 0 &&
        p.numConvGroups * p.inputChannelsPerConvGroup *
                std::size_t(w.inH) * w.inW * params.inputType.size() <
            (1ull << 31)) {
      plan.depthwiseWeightUpdate = true;
      mxk::DepthwiseDesc &f = plan.depthwiseForward;
      f.elemBytes = uint32_t(params.inputType.size());
      f.batch = uint32_t(p.inputChannelsPerConvGroup);
      f.channels = uint32_t(p.numConvGroups);
      f.inH = w.inH, f.inW = w.inW;
      f.outH = w.kH, f.outW = w.kW, f.kH = w.outH, f.kW = w.outW;
      f.padH = w.padH, f.padW = w.padW;
      f.strideH = w.dilH, f.strideW = w.dilW;
      f.dilH = w.strideH, f.dilW = w.strideW;
      f.loH = w.loH, f.hiH = w.hiH, f.loW = w.loW, f.hiW = w.hiW;
      // 3x3 layers that give every CU a band of rows: the persistent kernel
      // with the rows of both tensors in LDS rings (as for the forward pass)
      f.cus = gfx950::numCUs;
      const mxk::DepthwiseRowsLaunch l =
          mxk::depthwiseRowsDeltaLaunchShape(f);
      if (options.planConstraints.rowRing != 0 &&
          params.inputType == poplar::HALF &&
          mxk::depthwiseRowsDeltaTakes(f) &&
          (options.planConstraints.rowRing == 1 ||
           // (strips of fewer than four columns read mostly halo: N = 32,
           // 7 x 7, 960 channels 20.5 us against 13.1)
           (l.workgroups * 2 >= gfx950::numCUs && l.rowsOut >= 4 &&
            (l.colsOut >= 4 || l.strips == 1))))
        f.dense3x3 = 2;
    }
  }
  // The weight update pass of a dense layer with an undilated kernel and
  // input: batch = the layer's input channels, input channels = its batch,
  // kernel = its output field, output field = its kernel, kernel dilation =
  // its stride.  (Opt out:
  // planConstraints gfx950 kernel names one.)
  {
    const Simple2D w = asSimple2D(p);
    const int asked = options.planConstraints.weightDeltas;
    if (isWeightUpdatePass(options.pass) && asked != 0 && w.ok &&
        !w.hasDepth() && !w.outputPadded() && !w.kernelSelected &&
        !plan.zeroConv && !plan.depthwiseWeightUpdate && !w.inputDilated() &&
        w.batch == p.batchSize && w.strideH == 1 && w.strideW == 1 &&
        params.inputType == poplar::HALF &&
        (asked == 1 ||
         (options.planConstraints.kernel.empty() &&
          options.planConstraints.method == PlanConstraints::Method::ANY))) {
      mxk::WuTapDesc &f = plan.denseForward;
      f.batch = uint32_t(p.inputChannelsPerConvGroup);
      f.inH = w.inH, f.inW = w.inW;
      f.outH = w.kH, f.outW = w.kW, f.kH = w.outH, f.kW = w.outW;
      f.padH = w.padH, f.padW = w.padW;
      f.strideH = w.dilH, f.strideW = w.dilW; // (the layer's stride)
      f.loH = w.loH, f.hiH = w.hiH, f.loW = w.loW, f.hiW = w.hiW;
      f.groups = uint32_t(p.numConvGroups);
      f.ci = uint32_t(p.batchSize);
      f.co = uint32_t(p.outputChannelsPerConvGroup);
      f.chunkPixels = mxk::wuTapChunkPixels(f, gfx950::numCUs);
      // (enough pixels to be worth the matrix cores: a kernel-sized field
      // of a tiny batch stays with the general path)
      const std::size_t pixels = std::size_t(f.batch) * f.outH * f.outW;
      // ... and, in a grouped layer, channels that fill a quarter of the
      // kernel's 128 x 128 tile per (group, tap): every group brings its own
      // tiles, and poorly filled ones lose to the pass's own convolution
      // (N = 32, 28 x 28, 3 x 3: 32 groups of 16 -> 16 channels 420 against
      // 117 us, 8 groups of 32 -> 32 78 against 49, 2 groups of 64 -> 64 26
      // against 26.5, 4 groups of 64 -> 64 41 against 34 and 2 such groups on
      // 56 x 56 70 against 52; without groups 16 -> 16 on 56 x 56 ties at
      // 39 us and 32 -> 64 wins with 18 against 25).
      const std::size_t tileArea = std::size_t((f.ci + 127) / 128 * 128) *
                                   ((f.co + 127) / 128 * 128);
      const bool filled =
          f.groups == 1 || std::size_t(f.ci) * f.co * 4 > tileArea;
      const bool worth =
          pixels >= 1024 && f.ci >= 16 && f.co >= 16 && filled;
      plan.denseWeightUpdate = (asked == 1 || worth) && mxk::wuTapTakes(f);
    }
    if (asked == 1 && isWeightUpdatePass(options.pass) &&
        !plan.denseWeightUpdate && !plan.depthwiseWeightUpdate)
      throw poplar::invalid_option(
          "planConstraints gfx950 weightDeltas: no weight-delta kernel takes "
          "this layer's own tensors (half inputs, nothing dilated, truncated, "
          "padded or flipped on the kernel side, channels in whole 16-byte "
          "vectors)");
  }
  const auto &pc = options.planConstraints;
  if (convGroupsPerGroup > 1) {
    planned.numConvGroups /= convGroupsPerGroup;
    planned.inputChannelsPerConvGroup *= convGroupsPerGroup;
    planned.outputChannelsPerConvGroup *= convGroupsPerGroup;
  }
  const Simple2D s = asSimple2D(p);
  const bool halfIn = params.inputType == poplar::HALF;
  const bool quarterIn = params.inputType == poplar::QUARTER;
  const bool floatIn = params.inputType == poplar::FLOAT;
  const std::size_t ci = p.inputChannelsPerConvGroup;
  const std::size_t co = p.outputChannelsPerConvGroup;
  // The matrix-core kernel reads whole 16-byte vectors of channels; other
  // channel counts are padded with zeros (input: a copy per launch; weights:
  // when they are packed).
  const std::size_t vecElems = 16 / params.inputType.size();
  const std::size_t ciPadded = (ci + vecElems - 1) / vecElems * vecElems;

  // The matrix-core kernel addresses its input with 32-bit offsets from the
  // first image a tile reads.
  auto inputAddressable = [&] {
    mxk::IgemmDesc g{};
    g.batch = uint32_t(s.batch), g.groups = uint32_t(p.numConvGroups);
    g.inChansPerGroup = uint32_t(ciPadded);
    g.inD = s.inD, g.inH = s.inH, g.inW = s.inW;
    g.outD = s.outD, g.outH = s.outH, g.outW = s.outW;
    g.padD = s.padD, g.padH = s.padH, g.padW = s.padW;
    return s.batch < (1ull << 31) &&
           mxk::igemmAddressable(
               g, halfIn ? mxk::kHalf : floatIn ? mxk::kFloat : mxk::kQuarter);
  };

  // Which kernels can take this convolution at all?
  std::string igemmWhyNot, dwWhyNot;
  std::pair<unsigned, unsigned> dwTile{0, 0};
  if (plan.zeroConv)
    igemmWhyNot = dwWhyNot = "all outputs are zero";
  else if (!s.ok)
    igemmWhyNot = dwWhyNot = s.why;
  else {
    if (!(halfIn || quarterIn || floatIn))
      igemmWhyNot = "matrix-core kernel takes float, half or quarter inputs";
    else if (ciPadded != ci && (ci == 0 || (ci == 1 && co == 1)))
      // (one channel per group is vector-ALU work)
      igemmWhyNot = "input channels per group not a multiple of a 16-byte "
                    "vector";
    else if (ciPadded != ci && pc.kernel != "igemm" &&
             2.0 * double(s.batch) * s.outD * s.outH * s.outW * s.kD * s.kH *
                     s.kW * ci * co * p.numConvGroups <
                 double(1u << 22))
      igemmWhyNot = "too little work to pay for a padded copy of the input "
                    "(channels per group not a multiple of a 16-byte vector)";
    else if (std::size_t(s.outH) * s.strideH + std::size_t(s.kH) * s.dilH +
                     std::size_t(std::abs(s.padH)) >=
                 32768 ||
             std::size_t(s.outW) * s.strideW + std::size_t(s.kW) * s.dilW +
                     std::size_t(std::abs(s.padW)) >=
                 32768)
      igemmWhyNot = "field too large for 16-bit window origins";
    else if (s.hasDepth() &&
             ((s.inputDilated() &&
               !((s.inDilD == 1 || s.strideD == 1) &&
                 (s.inDilH == 1 || s.strideH == 1) &&
                 (s.inDilW == 1 || s.strideW == 1) &&
                 std::size_t(s.inDilD) * s.inDilH * s.inDilW <=
                     mxk::kIgemmMaxFused))))
      igemmWhyNot = "three field dimensions with a dilated input that does "
                    "not come apart into phases";
    else if (s.inputDilated() &&
             (std::size_t(s.inW) * p.getNumInputChans() *
                      params.inputType.size() >=
                  (1u << 24) ||
              s.inDilH >= (1u << 24) || s.inDilW >= (1u << 24)))
      igemmWhyNot = "input rows too long for the arithmetic tap addressing";
    else if (!s.inputDilated() && std::size_t(s.kD) * s.kH * s.kW > 32 &&
             (s.kD > 255 || s.kH > 255 || s.kW > 32767))
      igemmWhyNot = "kernel extent above 255 (32 767 in the last dimension)";
    else if (!inputAddressable() ||
             s.batch * s.outD * s.outH * s.outW >= (1ull << 31) ||
             p.numConvGroups * ((co + 127) / 128 * 128) * s.kD * s.kH * s.kW *
                     (ciPadded + vecElems * 8) * params.inputType.size() >=
                 (1ull << 31))
      igemmWhyNot = "tensor too large for 32-bit buffer addressing";
    if (s.hasDepth())
      dwWhyNot = "three field dimensions";
    else if (s.kernelSelected)
      dwWhyNot = "kernel truncation, padding or flip";
    else if (s.outputPadded())
      dwWhyNot = "output padding";
    else if (quarterIn && s.inputDilated())
      dwWhyNot = "depthwise kernel takes a dilated input as half or float";
    else if (ci != 1 || co != 1)
      dwWhyNot = "not one channel per group";
    else if (p.numConvGroups % vecElems != 0)
      dwWhyNot = "channel count not a multiple of a 16-byte vector";
    else if (std::size_t(s.inH) * s.inW * p.numConvGroups *
                     params.inputType.size() >=
                 (1ull << 30) ||
             std::size_t(s.outH) * s.outW * p.numConvGroups * 4 >=
                 (1ull << 30))
      dwWhyNot = "image too large for 32-bit buffer addressing";
    else if (!s.inputDilated() &&
             (dwTile = chooseDepthwiseTile(s, p.numConvGroups / vecElems))
                     .first == 0)
      dwWhyNot = "input patch of a single output pixel exceeds the LDS budget";

  }

  // Choose.  PopLibs method names map onto the kernels that take their role:
  // AMP -> matrix cores; HMAC / VMAC / SLIC -> vector-ALU direct kernel.
  Kernel chosen = Kernel::GENERIC;
  std::string reason;
  auto require = [&](const std::string &whyNot, const char *what) {
    if (!whyNot.empty())
      throw poplar::invalid_option(
          std::string("planConstraints ask for the ") + what +
          " kernel, which cannot take this convolution: " + whyNot);
  };
  if (pc.kernel == "generic") {
    reason = "forced by planConstraints";
  } else if (pc.kernel == "igemm") {
    require(igemmWhyNot, "igemm");
    chosen = Kernel::IGEMM;
    reason = "forced by planConstraints";
  } else if (pc.kernel == "depthwise") {
    require(dwWhyNot, "depthwise");
    chosen = Kernel::DEPTHWISE;
    reason = "forced by planConstraints";
  } else if (pc.method == Method::AMP && igemmWhyNot.empty()) {
    chosen = Kernel::IGEMM;
    reason = "method AMP -> matrix cores";
  } else if ((pc.method == Method::HMAC || pc.method == Method::VMAC ||
              pc.method == Method::SLIC) &&
             dwWhyNot.empty()) {
    chosen = Kernel::DEPTHWISE;
    reason = "method " + std::string(pc.method == Method::HMAC   ? "HMAC"
                                     : pc.method == Method::VMAC ? "VMAC"
                                                                 : "SLIC") +
             " -> vector-ALU direct kernel";
  } else if (pc.method == Method::HMAC || pc.method == Method::VMAC ||
             pc.method == Method::SLIC || pc.method == Method::OUTER_PRODUCT) {
    reason = "vector-ALU method requested; generic direct kernel";
  } else if (dwWhyNot.empty()) {
    chosen = Kernel::DEPTHWISE;
    reason = "one channel per group: memory-bound, vector-ALU direct kernel";
  } else if (igemmWhyNot.empty()) {
    chosen = Kernel::IGEMM;
    reason = "dense channels: implicit GEMM on the matrix cores";
  } else {
    reason = "generic direct kernel (" + igemmWhyNot + ")";
  }
  // An input of 1 to 4 channels (an image, a waveform): the matrix-core
  // kernel that takes the kW * Ci neighbouring elements under a kernel row in
  // chunks of 8, four to a k-step, instead of padding the channels to a whole
  // vector - no copy of the input, K = 192 instead of 392 for N = 32,
  // 224 x 224, 7 x 7 stride 2, 3 -> 64 (58 -> 19 us).
  {
    mxk::ThinInputDesc &t = plan.thinInput;
    t.batch = uint32_t(s.batch), t.inChans = uint32_t(ci);
    t.outChans = uint32_t(co);
    t.inH = s.inH, t.inW = s.inW, t.outH = s.outH, t.outW = s.outW;
    t.kH = s.kH, t.kW = s.kW, t.padH = s.padH, t.padW = s.padW;
    t.strideH = s.strideH, t.strideW = s.strideW;
    t.loH = s.loH, t.hiH = s.hiH, t.loW = s.loW, t.hiW = s.hiW;
    const bool shapeOk =
        !plan.zeroConv && s.ok && !s.hasDepth() && !s.inputDilated() &&
        !s.kernelSelected && !s.outputPadded() && s.dilH == 1 &&
        s.dilW == 1 && p.numConvGroups == 1 && s.batch < (1ull << 31) &&
        mxk::thinInputTakes(t,
                            halfIn    ? mxk::kHalf
                            : floatIn ? mxk::kFloat
                                      : mxk::kQuarter,
                            params.outputType == poplar::HALF ? mxk::kHalf
                                                              : mxk::kFloat);
    const bool unconstrained =
        pc.kernel.empty() && !pc.blockM && !pc.blockN && !pc.blockK &&
        !pc.splitK && !pc.stages && pc.patch < 1 && pc.pointwise != 1 &&
        (pc.method == Method::ANY || pc.method == Method::AMP);
    if (pc.thinInput == 1 && !shapeOk)
      throw poplar::invalid_option(
          "planConstraints gfx950 thinInput: that kernel takes 2-D "
          "convolutions of half inputs with 1 to 4 channels in one group "
          "(kW * Ci <= 32, at most 28 chunks of 8 elements over the kernel "
          "rows; 16, 32, 48 or 64 output "
          "channels; nothing dilated or flipped, no kernel truncation or "
          "padding, no output padding, no negative padding of the columns)");
    if (shapeOk && pc.thinInput != 0 &&
        (pc.thinInput == 1 || (unconstrained && chosen == Kernel::IGEMM))) {
      plan.thinInputOn = true;
      if (chosen != Kernel::IGEMM)
        chosen = Kernel::IGEMM, reason = "forced by planConstraints";
      else
        reason = "few input channels: a kernel row's pixels as one k-step on "
                 "the matrix cores";
    }
  }
  plan.kernel = chosen;
  plan.reason = reason;

  if (plan.thinInputOn) {
    plan.weightPackedElems = mxk::thinInputPackedElems(plan.thinInput);
    plan.workspaceBytes = 0;
  } else if (chosen == Kernel::IGEMM) {
    mxk::IgemmDesc &g = plan.igemm;
    g.batch = uint32_t(s.batch);
    g.groups = uint32_t(p.numConvGroups);
    g.inChansPerGroup = uint32_t(ciPadded);
    g.inD = s.inD, g.outD = s.outD, g.kD = s.kD, g.padD = s.padD;
    g.strideD = s.strideD, g.dilD = s.dilD, g.loD = s.loD, g.hiD = s.hiD;
    g.outChansPerGroup = uint32_t(co);
    g.inH = s.inH, g.inW = s.inW, g.outH = s.outH, g.outW = s.outW;
    g.kH = s.kH, g.kW = s.kW, g.padH = s.padH, g.padW = s.padW;
    g.strideH = s.strideH, g.strideW = s.strideW;
    g.dilH = s.dilH, g.dilW = s.dilW;
    g.loH = s.loH, g.hiH = s.hiH, g.loW = s.loW, g.hiW = s.hiW;
    g.inDilH = s.inDilH, g.inDilW = s.inDilW;
    if (s.kernelSelected) {
      plan.kernelSelected = true;
      plan.igemmTaps = {s.fullKW,
                        s.selFirstH, s.selStepH, s.kH,
                        s.selFirstW, s.selStepW, s.kW,
                        s.fullKH, s.selFirstD, s.selStepD, s.kD};
    }
    if (s.outputPadded()) {
      // the convolution writes the inside of the padded field; the launch
      // fills the field with zeros (or the bias) first
      g.outFullH = s.outH + s.outPadLoH + s.outPadHiH;
      g.outFullW = s.outW + s.outPadLoW + s.outPadHiW;
      g.outFullD = s.outD + s.outPadLoD + s.outPadHiD;
      g.outOffH = s.outPadLoH, g.outOffW = s.outPadLoW;
      g.outOffD = s.outPadLoD;
      plan.outputPadded = true;
      plan.outputPadLoH = s.outPadLoH, plan.outputPadHiH = s.outPadHiH;
      plan.outputPadLoW = s.outPadLoW, plan.outputPadHiW = s.outPadHiW;
      plan.outputPadLoD = s.outPadLoD, plan.outputPadHiD = s.outPadHiD;
    }
    // Tile shape.  M = batch * outH * outW pixels, N = out channels of one
    // group, K = kH * kW * in channels.  A 128-pixel tile keeps the A
    // fragment reuse high; N is 128 unless the group has at most 64 output
    // channels, when a narrower tile avoids computing padding.
    g.blockM = pc.blockM ? pc.blockM : 128;
    g.blockN = pc.blockN ? pc.blockN : (co <= 64 ? 64 : 128);
    const unsigned stepElems = unsigned(128 / params.inputType.size());
    g.blockK = pc.blockK ? pc.blockK : stepElems;
    // More than 64 output channels on few pixels (the deep 1 x 1 layers at
    // the end of a ResNet): 128 x 128 tiles leave CUs idle or need K split
    // over workgroups with a second kernel; twice as many 128 x 64 tiles, two
    // workgroups to a CU, fill the chip with K whole.  Weighed by the same
    // estimates (N = 32, 14 x 14, 1024 -> 256: 8.9 -> 7.1 us; 7 x 7, 2048 ->
    // 512: 12.8 -> 10.2; but 14 x 14, 1024 -> 512, 392 narrow tiles: 10.2
    // against 12.1, and the estimate keeps the wide tile there).
    bool narrowWhole = false;    // ... chosen: K stays whole
    std::size_t narrowSplit = 0; // ... or narrow tiles with K in this many parts
    if (!pc.blockN && !pc.splitK && !pc.stages && co > 64 &&
        g.blockM == 128) {
      const std::size_t m = s.batch * s.outD * s.outH * s.outW;
      const std::size_t mTiles = (m + 127) / 128;
      const std::size_t kSteps =
          (std::size_t(s.kD) * s.kH * s.kW * ciPadded + stepElems - 1) /
          stepElems;
      const std::size_t wide = mTiles * ((co + 127) / 128) * p.numConvGroups;
      const std::size_t narrow = mTiles * ((co + 63) / 64) * p.numConvGroups;
      std::size_t parts = 1;
      if (wide != 0 && wide * 2 <= gfx950::numCUs && kSteps >= 16)
        parts = std::max<std::size_t>(
            1, std::min<std::size_t>(gfx950::numCUs / wide, kSteps / 4));
      const std::size_t partial =
          parts * m * p.numConvGroups * ((co + 127) / 128 * 128) * 4;
      const double wideUs = std::min(
          estimateStreaming(wide, kSteps, wide > gfx950::numCUs ? 2 : 1, 128,
                            1, 0),
          parts > 1 ? estimateStreaming(wide * parts,
                                        (kSteps + parts - 1) / parts, 1, 128,
                                        unsigned(parts), partial)
                    : 1e30);
      const double wideWholeUs = estimateStreaming(
          wide, kSteps, wide > gfx950::numCUs ? 2 : 1, 128, 1, 0);
      if (estimateStreaming(narrow, kSteps, 2, 64, 1, 0) < wideUs) {
        g.blockN = 64, narrowWhole = true;
      } else if (wideUs < wideWholeUs && narrow * 2 <= gfx950::numCUs) {
        // K split wins: then over narrow tiles, in half as many parts of at
        // least 8 k-steps - the same number of workgroups, each with half the
        // weights to fetch per k-step and half the fp32 tile to write, and
        // half the partial tiles in all.  Measured for skinny products and
        // deep layers alike (wide -> narrow, us): 32 x 4096 x 4096 13.3 ->
        // 11.4, 256 x 4096 x 1024 17.5 -> 12.2, 512 x 4096 x 1024 18.1 ->
        // 14.2, N = 8 7 x 7 3 x 3 512 -> 512 15.2 -> 11.0, N = 1 9.9 -> 8.4;
        // level where the rule already chose few parts (N = 32 7 x 7 3 x 3
        // 512 -> 512 19.0 -> 18.6, 14 x 14 stride 2 18.2 -> 18.4).
        const std::size_t narrowParts = std::min<std::size_t>(
            gfx950::numCUs / narrow, kSteps / 8);
        if (narrowParts > 1)
          g.blockN = 64, narrowSplit = narrowParts;
      }
    }
    const bool anyHeight = pc.patch == 2 && g.blockM >= 1 && g.blockM <= 112;
    if ((g.blockM != 128 && g.blockM != 64 && !anyHeight) ||
        (g.blockN != 64 && g.blockN != 128) ||
        g.blockK != stepElems)
      throw poplar::invalid_option(
          "planConstraints gfx950 tile not available: blockM must be 128 (64 "
          "with patch 1, 1 to 112 with patch 2), blockN 64 or 128, blockK 32 "
          "(float), 64 (half) or 128 (quarter)");
    const std::size_t k = std::size_t(s.kD) * s.kH * s.kW * ciPadded;
    plan.coPadded = (co + g.blockN - 1) / g.blockN * g.blockN;
    plan.kPadded = (k + g.blockK - 1) / g.blockK * g.blockK;
    plan.weightPackedElems = p.numConvGroups * plan.coPadded * plan.kPadded;
    // Too few output tiles to fill the chip but a long K (a weight update
    // pass, a skinny matrix product): cut K into parts, one workgroup each,
    // as many as bring the grid up to about one workgroup per CU while every
    // part keeps at least 4 k-steps; the fp32 partial tiles go through a
    // workspace (the role of PopLibs' in-channel split with ReduceAdd,
    // lib/poplin/ConvReduce.cpp:316-362).
    {
      const std::size_t m = s.batch * s.outD * s.outH * s.outW;
      const std::size_t tiles = ((m + g.blockM - 1) / g.blockM) *
                                (plan.coPadded / g.blockN) * p.numConvGroups;
      const std::size_t kSteps = plan.kPadded / g.blockK;
      std::size_t parts = 1;
      if (pc.splitK)
        parts = pc.splitK;
      else if (narrowSplit)
        parts = narrowSplit;
      else if (!narrowWhole && tiles != 0 && tiles * 2 <= gfx950::numCUs &&
               kSteps >= 16)
        parts = std::min<std::size_t>(gfx950::numCUs / tiles, kSteps / 4);
      parts = std::max<std::size_t>(1, std::min(parts, kSteps));
      // ... where that is estimated to pay for the partial tiles' round trip
      // and the second kernel: N = 32, 14 x 14, 1 x 1, 1024 -> 256 channels
      // (98 tiles of 16 k-steps) 16.4 us in two parts, 8.9 us whole; 7 x 7,
      // 3 x 3, 512 -> 512 (52 tiles of 72 k-steps) 18.7 in four, 21.1 whole.
      if (!pc.splitK && !narrowSplit && parts > 1 &&
          estimateStreaming(tiles, kSteps, g.blockN == 64 ? 2 : 1, g.blockN, 1,
                            0) <=
              estimateStreaming(tiles * parts, (kSteps + parts - 1) / parts,
                                1, g.blockN, unsigned(parts),
                                parts * m * p.numConvGroups * plan.coPadded *
                                    4))
        parts = 1;
      const std::size_t chans = p.numConvGroups * co;
      // partial tiles of more than 1 GB are not worth it
      if (parts * m * chans * 4 > (1ull << 30))
        parts = 1;
      // (the sum of the parts is written pixel after pixel: not into a
      // padded output field)
      if (s.outputPadded())
        parts = 1;
      // (three dimensions over a dilated input run as phases only)
      if (s.hasDepth() && s.inputDilated())
        parts = 1;
      g.splitK = uint32_t(parts);
      plan.workspaceBytes = mxk::igemmWorkspaceBytes(g);
      if (ciPadded != ci) {
        plan.paddedInputChans = ciPadded;
        plan.paddedInputOffset = (plan.workspaceBytes + 255) / 256 * 256;
        plan.workspaceBytes = plan.paddedInputOffset +
                              s.batch * s.inD * s.inH * s.inW *
                                  p.numConvGroups * ciPadded *
                                  params.inputType.size();
      }
      // More workgroups than CUs: run the 128-wide tile with two LDS stages
      // instead of four, so that two workgroups share a CU and one's
      // start-up, barriers and epilogue are covered by the other's MFMAs.
      // With one workgroup per CU or fewer the deeper prefetch is worth
      // more.
      g.stages = pc.stages ? pc.stages
                           : (tiles * parts > gfx950::numCUs ? 2 : 4);
      if (g.stages != 2 && g.stages != 4)
        throw poplar::invalid_option(
            "planConstraints gfx950 stages must be 2 or 4");
    }
    // Zero-stuffed input, window moving by single pixels: one ordinary
    // convolution per phase instead of arithmetic on every tap - no MACs on
    // the stuffed zeros, and the fast tap-mask addressing.
    if (s.inputDilated() && g.splitK == 1 &&
        (s.inDilD == 1 || s.strideD == 1) &&
        (s.inDilH == 1 || s.strideH == 1) &&
        (s.inDilW == 1 || s.strideW == 1) &&
        std::size_t(s.inDilD) * s.inDilH * s.inDilW <= mxk::kIgemmMaxFused) {
      // One dimension of one phase.  The window of output o = q * inDil +
      // phase meets real input under kernel tap k when phase - pad + k * dil
      // is a multiple of inDil - taps first, first + step, ... - and reads
      // input q + (phase - pad + k * dil) / inDil there.
      struct Dim {
        uint32_t out = 0, first = 0, step = 1, count = 0;
        int32_t pad = 0;
        uint32_t dil = 1;
        bool dead = false; // no tap ever meets real input: all zeros
      };
      auto dimOf = [](uint32_t phase, uint32_t inDil, uint32_t out,
                      uint32_t k, int32_t pad, uint32_t dil) {
        Dim r;
        r.out = out > phase ? (out - phase + inDil - 1) / inDil : 0;
        int64_t firstOffset = 0;
        for (uint32_t t = 0; t != k; ++t) {
          const int64_t x = int64_t(phase) - pad + int64_t(t) * dil;
          if (x % int64_t(inDil) != 0)
            continue;
          if (r.count == 0)
            r.first = t, firstOffset = x / int64_t(inDil);
          else if (r.count == 1)
            r.step = t - r.first;
          ++r.count;
        }
        if (r.count == 0) {
          r.dead = true, r.count = 1;
          return r;
        }
        r.pad = int32_t(-firstOffset);
        r.dil = r.count > 1 ? r.step * dil / inDil : 1;
        return r;
      };
      std::size_t offset = 0;
      for (uint32_t pd = 0; pd != s.inDilD; ++pd)
      for (uint32_t ph = 0; ph != s.inDilH; ++ph)
        for (uint32_t pw = 0; pw != s.inDilW; ++pw) {
          // a dimension that is not dilated keeps its stride and geometry
          const Dim dd = s.inDilD == 1
                             ? Dim{s.outD, 0, 1, s.kD, s.padD, s.dilD, false}
                             : dimOf(pd, s.inDilD, s.outD, s.kD, s.padD,
                                     s.dilD);
          const Dim h = s.inDilH == 1
                            ? Dim{s.outH, 0, 1, s.kH, s.padH, s.dilH, false}
                            : dimOf(ph, s.inDilH, s.outH, s.kH, s.padH, s.dilH);
          const Dim w = s.inDilW == 1
                            ? Dim{s.outW, 0, 1, s.kW, s.padW, s.dilW, false}
                            : dimOf(pw, s.inDilW, s.outW, s.kW, s.padW, s.dilW);
          if (dd.out == 0 || h.out == 0 || w.out == 0)
            continue;
          mxconv_plan::IgemmPhase phase;
          mxk::IgemmDesc &q = phase.d;
          q = g;
          q.inDilH = q.inDilW = 1;
          q.outH = h.out, q.outW = w.out, q.kH = h.count, q.kW = w.count;
          q.padH = h.pad, q.padW = w.pad, q.dilH = h.dil, q.dilW = w.dil;
          q.outD = dd.out, q.kD = dd.count, q.padD = dd.pad, q.dilD = dd.dil;
          if (s.inDilD != 1)
            q.strideD = 1;
          if (dd.dead)
            q.loD = q.hiD = 0;
          q.outFullD = s.outD + s.outPadLoD + s.outPadHiD;
          q.outStepD = s.inDilD, q.outOffD = pd + s.outPadLoD;
          if (s.inDilH != 1)
            q.strideH = 1;
          if (s.inDilW != 1)
            q.strideW = 1;
          if (h.dead)
            q.loH = q.hiH = 0;
          if (w.dead)
            q.loW = q.hiW = 0;
          q.outFullH = s.outH + s.outPadLoH + s.outPadHiH;
          q.outFullW = s.outW + s.outPadLoW + s.outPadHiW;
          q.outStepH = s.inDilH, q.outStepW = s.inDilW;
          q.outOffH = ph + s.outPadLoH, q.outOffW = pw + s.outPadLoW;
          const bool dead = dd.dead || h.dead || w.dead;
          q.noTaps = dead ? 1 : 0;
          // (tap j of the phase is tap first + j * step of the applied
          // kernel, which is a selection of the stored one itself)
          phase.taps = {s.fullKW,
                        s.selFirstH + s.selStepH * h.first,
                        s.selStepH * h.step,
                        dead ? 0u : h.count,
                        s.selFirstW + s.selStepW * w.first,
                        s.selStepW * w.step,
                        dead ? 0u : w.count,
                        s.fullKH,
                        s.selFirstD + s.selStepD * dd.first,
                        s.selStepD * dd.step,
                        dead ? 0u : dd.count};
          const std::size_t kk =
              std::size_t(q.kD) * q.kH * q.kW * ciPadded;
          phase.kPadded = (kk + g.blockK - 1) / g.blockK * g.blockK;
          phase.packedOffset = offset;
          offset += p.numConvGroups * plan.coPadded * phase.kPadded;
          plan.igemmPhases.push_back(phase);
        }
      // (kernel of more than 32 taps per phase: the ranges take over inside
      // the kernel, as for any convolution)
      plan.weightPackedElems = offset;
      std::size_t phaseTiles = 0;
      for (const auto &ph : plan.igemmPhases)
        phaseTiles += (std::size_t(ph.d.batch) * ph.d.outD * ph.d.outH *
                           ph.d.outW +
                       g.blockM - 1) /
                      g.blockM * (plan.coPadded / g.blockN) * g.groups;
      const uint32_t stages =
          pc.stages ? pc.stages : (phaseTiles > gfx950::numCUs ? 2 : 4);
      for (auto &ph : plan.igemmPhases)
        ph.d.stages = stages;
      g.stages = stages;
    }
    // A pointwise convolution with few input channels is bound by HBM, not
    // by the matrix cores: unless the big tile was asked for explicitly, the
    // streaming kernel of small workgroups takes it.
    mxk::PointwiseDesc &pw = plan.pointwise;
    pw.batch = g.batch, pw.pixels = s.outH * s.outW;
    pw.groups = g.groups, pw.inChansPerGroup = g.inChansPerGroup;
    pw.outChansPerGroup = g.outChansPerGroup;
    pw.chanTiles = pc.chanTiles;
    pw.elemBytes = uint32_t(params.inputType.size());
    const bool unitWindow =
        !s.hasDepth() && !s.outputPadded() && !s.kernelSelected &&
        !s.inputDilated() &&
        g.splitK == 1 && s.kH == 1 &&
        s.kW == 1 &&
        s.strideH == 1 && s.strideW == 1 &&
        s.padH == 0 && s.padW == 0 && s.loH == 0 && s.loW == 0 &&
        s.hiH == s.inH && s.hiW == s.inW && s.outH == s.inH &&
        s.outW == s.inW;
    // (The kernel runs 136 to 248 input channels as rows of 256, up to 44 %
    // of them padding it multiplies and makes room for: the big tile is
    // faster on small layers - N = 32, 28 x 28, 144 -> 32: 4.6 against 5.3 us,
    // 192 -> 32: 4.6 against 5.4, 7 x 7, 160 -> 960: 4.8 against 5.5 - and
    // slower on large ones: 56 x 56, 144 -> 24: 11.9 against 8.9.)
    // (fp8 rows count by their bytes: two channels for one of fp16)
    const std::size_t rowChans = ci * params.inputType.size() / 2;
    const bool paddedSmall = rowChans > 128 && rowChans < 256 &&
                             std::size_t(pw.batch) * pw.pixels < 65536 &&
                             pc.pointwise != 1;
    // (fp8 rows of 512 bytes or more: the kernel's MFMAs take 16 channels at
    // a time whatever the type, so deep fp8 layers are the matrix cores' -
    // N = 32, 28 x 28, 512 -> 128: 7.4 us against the big tile's 6.5,
    // N = 64, 14 x 14, 1024 -> 256: 8.5 against 7.8; with 256 channels and
    // fewer it wins, 14 x 14, 256 -> 1024: 10.0 against 12.2, 56 x 56,
    // 256 -> 64: 8.4 against 11.0, 112 x 112, 32 -> 64: 14.6 against 24.1)
    const bool deepQuarter =
        quarterIn && ci >= 512 && pc.pointwise != 1;
    plan.pointwiseOn =
        unitWindow && ciPadded == ci && !paddedSmall && !deepQuarter &&
        (pc.kernel != "igemm" || pc.pointwise == 1) && pc.pointwise != 0 &&
        pc.patch < 1 && !pc.blockM &&
        !pc.blockN && !pc.blockK &&
        mxk::pointwiseTakes(pw,
                            halfIn    ? mxk::kHalf
                            : floatIn ? mxk::kFloat
                                      : mxk::kQuarter,
                            params.outputType == poplar::HALF ? mxk::kHalf
                                                              : mxk::kFloat);
    if (plan.pointwiseOn)
      plan.weightPackedElems = mxk::pointwisePackedElems(pw);
    else if (pc.pointwise == 1)
      throw poplar::invalid_option(
          "planConstraints gfx950 pointwise: that kernel takes 1x1, unit "
          "stride, unpadded convolutions of half inputs with a multiple of 8 "
          "up to 512 input channels per group (quarter inputs: a multiple of "
          "16 up to 1024), with no other tile constraint");
    else if (pc.chanTiles)
      throw poplar::invalid_option(
          "planConstraints gfx950 chanTiles: the pointwise streaming kernel "
          "does not take this convolution with that many 64-channel tiles "
          "per workgroup (they divide the layer's; at most 4 with up to 64 "
          "input channels, 2 with up to 256, 1 beyond)");
    // Unit stride and whole 128-byte slices of channels: the kernel that
    // keeps the tile's input patch in LDS reads every input element once
    // instead of once per tap.
    if (!plan.pointwiseOn && plan.igemmPhases.empty() &&
        !plan.paddedInputChans &&
        (g.splitK == 1 || !pc.splitK) && pc.patch != 0 &&
        !pc.blockN && !pc.blockK && !pc.stages) {
      const int inId = halfIn ? mxk::kHalf : floatIn ? mxk::kFloat
                                                     : mxk::kQuarter;
      const int outId =
          params.outputType == poplar::HALF ? mxk::kHalf : mxk::kFloat;
      const std::size_t m = std::size_t(s.batch) * s.outH * s.outW;
      const std::size_t nTiles128 = (co + 127) / 128 * p.numConvGroups;
      const std::size_t stepBytes = 128;
      const std::size_t patchSteps =
          ciPadded * params.inputType.size() / stepBytes * s.kH * s.kW;
      // Weigh the tilings by estimated time: the streaming kernel as planned
      // above against this kernel with tiles of 128 and 64 pixels (32-pixel
      // MFMA blocks) and with the layer cut into as many equal tiles of at
      // most 112 pixels as there are CUs (16-pixel blocks).
      struct Tiling {
        uint32_t patch, blockM;
      };
      std::vector<Tiling> tilings;
      auto add = [&](const std::string &name, Tiling tiling,
                     std::size_t workgroups, std::size_t perCU,
                     std::size_t kSteps, double us, double rounds) {
        mxconv_plan::Candidate c;
        c.name = name, c.workgroups = workgroups, c.perCU = perCU;
        c.kSteps = kSteps, c.estimateUs = us, c.rounds = rounds;
        plan.candidates.push_back(c);
        tilings.push_back(tiling);
        return plan.candidates.size() - 1;
      };
      const std::size_t none = ~std::size_t(0);
      auto addPatch = [&](uint32_t mode, uint32_t bm) -> std::size_t {
        mxk::IgemmDesc t = g;
        t.patch = mode, t.blockM = bm;
        t.splitK = 1; // (asked for by name, it runs K whole)
        if (!mxk::igemmPatchTakes(t, inId, outId))
          return none;
        const std::size_t tiles = (m + bm - 1) / bm * nTiles128;
        return add("resident patch " + std::to_string(bm) + " x 128" +
                       (mode == 2 ? ", 16-pixel blocks" : ""),
                   Tiling{mode, bm}, tiles, 1, patchSteps,
                   estimatePatch(tiles, patchSteps, mode, bm),
                   roundsOf(tiles, 1));
      };
      // Equal tiles, one per CU, in whole 16-pixel MFMA blocks - a tile of 98
      // pixels costs its workgroup the seven blocks a tile of 112 does, and
      // 224 workgroups of 112 are through sooner than 256 of 98 (c2: 8.7
      // against 9.1 us); 112 pixels where that takes several rounds.
      const std::size_t across = gfx950::numCUs / std::max<std::size_t>(
                                                      1, nTiles128);
      const uint32_t equalM =
          across == 0
              ? 112u
              : uint32_t(std::min<std::size_t>(
                    112, ((m + across - 1) / across + 15) / 16 * 16));
      const std::size_t streamTiles =
          (m + 127) / 128 * (plan.coPadded / g.blockN) * p.numConvGroups *
          g.splitK;
      const std::size_t streamSteps =
          (plan.kPadded / g.blockK + g.splitK - 1) / g.splitK;
      const std::size_t streamPerCU = g.blockN == 64 || g.stages == 2 ? 2 : 1;
      const std::size_t iStream =
          add("streaming 128 x " + std::to_string(g.blockN) + ", " +
                  std::to_string(g.blockN == 128 ? g.stages : 3) + " stages" +
                  (g.splitK > 1 ? ", K in " + std::to_string(g.splitK) +
                                      " parts"
                                : ""),
              Tiling{0, 128}, streamTiles, streamPerCU, streamSteps,
              estimateStreaming(streamTiles, streamSteps, streamPerCU,
                                g.blockN, g.splitK,
                                mxk::igemmWorkspaceBytes(g)),
              roundsOf(streamTiles, streamPerCU));
      std::size_t best = iStream;
      if (pc.patch >= 1) {
        // planConstraints: whenever the kernel can, with the tile asked for
        const uint32_t bm = pc.blockM ? pc.blockM
                                      : pc.patch == 2 ? equalM : 128u;
        const std::size_t i = addPatch(uint32_t(pc.patch), bm);
        if (i != none)
          best = i;
      } else if (s.kH * s.kW > 1 && co > 64) {
        // (also against a streaming plan that splits K: the patch kernel's
        // equal tiles fill the chip without the second kernel - N = 32,
        // 14 x 14, 256 -> 256 channels 20.4 -> 12.4 us, N = 8, 28 x 28,
        // 128 -> 128 15.0 -> 7.7)
        for (Tiling t : {Tiling{1, 128}, Tiling{1, 64}, Tiling{2, equalM}}) {
          // (a forced tile height picks among the patch tilings only)
          if (pc.blockM && pc.blockM != t.blockM)
            continue;
          const std::size_t i = addPatch(t.patch, t.blockM);
          if (i != none && plan.candidates[i].estimateUs <
                               plan.candidates[best].estimateUs)
            best = i;
        }
      }
      plan.candidates[best].chosen = true;
      if (best != iStream) {
        g.patch = tilings[best].patch;
        g.blockM = tilings[best].blockM;
        g.splitK = 1;
        g.blockN = 128;
        g.patchMaxRows = 0;
        g.patchMaxRows = mxk::igemmPatchMaxRows(g);
        plan.workspaceBytes = 0;
        plan.coPadded = (co + 127) / 128 * 128;
        plan.weightPackedElems = mxk::igemmPatchPackedElems(g, inId);
      }
    }
    if (!g.patch && g.blockM != 128)
      throw poplar::invalid_option(
          "planConstraints gfx950 blockM 64 goes with the resident-patch "
          "kernel only");
  } else if (chosen == Kernel::DEPTHWISE) {
    mxk::DepthwiseDesc &d = plan.depthwise;
    d.batch = uint32_t(s.batch);
    d.channels = uint32_t(p.numConvGroups);
    d.inH = s.inH, d.inW = s.inW, d.outH = s.outH, d.outW = s.outW;
    d.kH = s.kH, d.kW = s.kW, d.padH = s.padH, d.padW = s.padW;
    d.strideH = s.strideH, d.strideW = s.strideW;
    d.dilH = s.dilH, d.dilW = s.dilW;
    d.loH = s.loH, d.hiH = s.hiH, d.loW = s.loW, d.hiW = s.hiW;
    d.tileH = dwTile.first, d.tileW = dwTile.second;
    d.inDilH = s.inDilH, d.inDilW = s.inDilW;
    d.elemBytes = uint32_t(params.inputType.size());
    const int dwType = halfIn ? mxk::kHalf
                       : floatIn ? mxk::kFloat
                                 : mxk::kQuarter;
    // 7 x 7 taps at unit stride: a thread forms a strip of neighbouring
    // pixels, and the tile is chosen to fill the workgroup's 256 threads.
    if (mxk::depthwiseStripTakes(d) && !(pc.tileH || pc.tileW))
      chooseDepthwiseStripTile(d);
    // An explicit tile asks for the LDS-tiled kernel.
    d.dense3x3 = !s.inputDilated() && !(pc.tileH || pc.tileW) &&
                 mxk::depthwise3x3Takes(d, dwType);
    // Layers that give every CU a band of at least four output rows go to
    // the persistent kernel with a ring of input rows in LDS: its start-up
    // (seven rows before the first output; 3.5 us for the smallest layer
    // against 2.9 us) wants rows to spread over.  Layers of more channels
    // than the small-workgroup kernel takes (224) always do: the kernel of
    // LDS halo tiles needs 5 to 8 us for the smallest of them.
    if (!s.inputDilated() && !(pc.tileH || pc.tileW) && pc.rowRing != 0) {
      d.cus = gfx950::numCUs;
      const mxk::DepthwiseRowsLaunch l = mxk::depthwiseRowsLaunchShape(d);
      const bool takes = mxk::depthwiseRowsTakes(d, dwType);
      if (pc.rowRing == 1 && !takes)
        throw poplar::invalid_option(
            "planConstraints gfx950 rowRing: that kernel takes 3x3 or 5x5 "
            "taps, stride 1 or 2, channels in vectors of 8, at most 2048 "
            "(5x5: 1224) to a pixel");
      // 5 x 5 taps (25 multiply-adds per output and channel: the vector ALU
      // shares the bound): strips of four columns or more, and at stride 2
      // bands of six rows or more - N = 32, 56 x 56, 144 channels, stride 2
      // 26.0 -> 13.1 us and 14 x 14, 480 channels 14.7 -> 9.3, but 28 x 28,
      // 240 channels, stride 2 8.1 -> 9.3 and 7 x 7, 1152 channels (strips of
      // one column) 10.6 -> 12.6.
      const bool five = d.kH == 5;
      const bool fiveWorth = (l.colsOut >= 4 || l.strips == 1) &&
                             (d.strideH == 1 || l.rowsOut >= 6);
      if (takes &&
          (pc.rowRing == 1 ||
           (five ? fiveWorth
                 : !d.dense3x3 || (l.workgroups * 2 >= gfx950::numCUs &&
                                   l.rowsOut >= 4))))
        d.dense3x3 = 2;
    } else if (pc.rowRing == 1) {
      throw poplar::invalid_option(
          "planConstraints gfx950 rowRing: the layer is not one the "
          "depthwise 3x3 kernels take");
    }
    if (!s.inputDilated() && (pc.tileH || pc.tileW)) {
      d.tileH = pc.tileH ? pc.tileH : d.tileH;
      d.tileW = pc.tileW ? pc.tileW : d.tileW;
      if (mxk::depthwiseStripTakes(d))
        d.stripPixels = stripPixelsFor(d, d.tileH, d.tileW);
      if (mxk::depthwiseTileLdsBytes(d) >
          (d.stripPixels ? mxk::kDepthwiseTileLdsMost : 64 * 1024))
        throw poplar::invalid_option(
            "planConstraints gfx950 tileH x tileW: the input patch of such a "
            "tile does not fit 64 KB of LDS");
    }
    plan.weightPackedElems = plan.weightElems; // [kH*kW][C]
  } else {
    plan.weightPackedElems = plan.weightElems; // [G][K][Ci][Co]
  }
  if (convGroupsPerGroup > 1 && chosen == Kernel::IGEMM) {
    plan.convGroupsPerGroup = convGroupsPerGroup;
    plan.weightExpandElems = plan.weightElems * convGroupsPerGroup;
  }
  return plan;
}

} // namespace

} // namespace poplin

std::string mxconv_plan::constraintsJson() const {
  std::ostringstream os;
  os << "{";
  if (wuGroupsPerGroup > 1 ||
      (madeForWeightUpdate && canonical.numConvGroups > 1))
    os << "\"convGroupsPerGroup\": " << wuGroupsPerGroup << ", ";
  else if (kernel == Kernel::IGEMM && canonical.numConvGroups > 1)
    os << "\"convGroupsPerGroup\": " << convGroupsPerGroup << ", ";
  os << "\"gfx950\": {";
  switch (kernel) {
  case Kernel::GENERIC:
    os << "\"kernel\": \"generic\"";
    break;
  case Kernel::DEPTHWISE:
    os << "\"kernel\": \"depthwise\", \"rowRing\": "
       << (depthwise.dense3x3 == 2 ? 1 : 0);
    // (an explicit tile names the LDS-tiled kernel)
    if (!depthwise.dense3x3 && depthwise.inDilH == 1 && depthwise.inDilW == 1)
      os << ", \"tileH\": " << depthwise.tileH << ", \"tileW\": "
         << depthwise.tileW;
    break;
  case Kernel::IGEMM:
    os << "\"kernel\": \"igemm\"";
    if (thinInputOn) {
      os << ", \"thinInput\": 1";
    } else if (pointwiseOn) {
      os << ", \"pointwise\": 1, \"chanTiles\": "
         << mxk::pointwiseLaunchShape(pointwise, gfx950::numCUs).chansPerWorkgroup / 64;
    } else if (igemm.patch) {
      os << ", \"pointwise\": 0, \"patch\": " << igemm.patch
         << ", \"blockM\": " << igemm.blockM;
    } else {
      os << ", \"pointwise\": 0, \"patch\": 0, \"blockM\": "
         << igemm.blockM << ", \"blockN\": " << igemm.blockN
         << ", \"blockK\": " << igemm.blockK << ", \"splitK\": "
         << igemm.splitK << ", \"stages\": " << igemm.stages;
    }
    break;
  }
  if (madeForWeightUpdate) {
    os << ", \"weightDeltas\": "
       << (weightUpdateProduct                           ? 2
           : denseWeightUpdate || depthwiseWeightUpdate ? 1
                                                        : 0);
    if (depthwiseWeightUpdate && kernel != Kernel::DEPTHWISE)
      os << ", \"rowRing\": " << (depthwiseForward.dense3x3 == 2 ? 1 : 0);
  }
  os << "}}";
  return os.str();
}

mxconv_plan::DetailedEstimate mxconv_plan::detailedEstimate() const {
  // Kernels that stream their tensors once (1x1 with few channels, depthwise,
  // fills) run at about 6.4 TB/s behind the launch: 64 MB in 11.6 us and
  // 96 MB in 17.9 us measured.
  constexpr double kStreamBytesPerUs = 6.4e6;
  auto streamed = [&](std::size_t bytes) {
    return poplin::kLaunchUs + double(bytes) / kStreamBytesPerUs;
  };
  auto spread = [](DetailedEstimate &e, std::size_t workgroups,
                   std::size_t perCU) {
    const std::size_t slots = std::size_t(gfx950::numCUs) * perCU;
    e.parallelSplit = std::max<std::size_t>(1, std::min(workgroups, slots));
    e.serialSplit =
        std::max<std::size_t>(1, (workgroups + slots - 1) / slots);
  };
  DetailedEstimate e;
  if (zeroConv) {
    e.computeUs = streamed(outputBytes());
    return e;
  }
  // A weight update pass that runs on the layer's own tensors: what those
  // kernels were measured at.  Matrix-core kernel + ordered sum, two
  // launches, about 350 TFLOP/s of the dense count while the loop waits for
  // its loads (N = 32, 28 x 28, 128 -> 128, 3 x 3: 24.5 us, of which the sum
  // of the chunks' 16.8 MB of fp32 tiles 5.2); depthwise rows + the sum of
  // the workgroups' tiles (4.5 us) behind one pass over both tensors (N = 32,
  // 112 x 112, 96 channels, stride 2: 20.4 us).
  if (weightUpdateProduct) {
    // the product as planned, behind the deltas' transpose and the packing
    // of the activations (each read once and written once)
    DetailedEstimate e = weightUpdateProduct->detailedEstimate();
    if (e.known) {
      e.rearrangementBytes += weightUpdateProduct->inputBytes() +
                              weightUpdateProduct->weightPackedBytes();
      e.rearrangementUs +=
          streamed(2 * weightUpdateProduct->inputBytes()) +
          streamed(2 * weightUpdateProduct->weightPackedBytes());
    }
    return e;
  }
  if (denseWeightUpdate) {
    const auto &f = denseForward;
    const double flops = 2.0 * f.batch * f.outH * f.outW * f.groups * f.ci *
                         f.co * f.kH * f.kW;
    const double all = 2 * poplin::kLaunchUs + flops / 3.5e8;
    e.reductionBytes = mxk::wuTapWorkspaceBytes(f);
    e.reductionUs = std::min(all / 2, streamed(e.reductionBytes));
    e.computeUs = all - e.reductionUs;
    const std::size_t m = std::size_t(f.batch) * f.outH * f.outW;
    spread(e,
           std::size_t(f.groups) * f.kH * f.kW * ((f.ci + 127) / 128) *
               ((f.co + 127) / 128) * ((m + f.chunkPixels - 1) / f.chunkPixels),
           1);
    return e;
  }
  if (depthwiseWeightUpdate) {
    const auto &f = depthwiseForward;
    const std::size_t bytes =
        (std::size_t(f.batch) * f.inH * f.inW + std::size_t(f.batch) * f.outH *
                                                     f.outW) *
        f.channels * 2;
    e.computeUs = streamed(bytes);
    e.reductionUs = 4.5;
    if (f.dense3x3 == 2) {
      e.reductionBytes = mxk::depthwiseRowsDeltaWorkspaceBytes(f);
      spread(e, mxk::depthwiseRowsDeltaLaunchShape(f).workgroups, 1);
    }
    return e;
  }
  switch (kernel) {
  case Kernel::GENERIC:
    e.known = false;
    return e;
  case Kernel::DEPTHWISE:
    e.computeUs = streamed(inputBytes() + outputBytes() + weightPackedBytes());
    if (depthwise.dense3x3 == 2)
      spread(e, mxk::depthwiseRowsLaunchShape(depthwise).workgroups, 1);
    break;
  case Kernel::IGEMM: {
    if (thinInputOn) {
      // Launch, weights and the first tile's rows (3.5 us), then the block
      // loop - matrix pipe and vector ALU take turns on a SIMD: 1.3 PFLOP/s
      // of the k-steps' padded work - and the tensors' bytes beside it, which
      // overlap it only in part.  Against measurements (N = 32, 224 x 224):
      // 7 x 7 stride 2 3 -> 64 17.9 for 19-21 us, 3 x 3 3 -> 64 37.5 for 35,
      // 3 x 3 3 -> 32 21.1 for 21.1, stride 2 8.7 for 9.5.
      const mxk::ThinInputLaunch l =
          mxk::thinInputLaunchShape(thinInput, gfx950::numCUs);
      const double flops = 2.0 * thinInput.batch * thinInput.outH *
                           ((thinInput.outW + 15) / 16 * 16) *
                           thinInput.outChans * 32.0 *
                           mxk::thinInputKSteps(thinInput);
      e.computeUs =
          3.5 + flops / 1.3e9 +
          double(inputBytes() + outputBytes() + weightPackedBytes()) / 9.0e6;
      spread(e, l.workgroups, 1);
      break;
    }
    if (pointwiseOn) {
      e.computeUs =
          streamed(inputBytes() + outputBytes() + weightPackedBytes());
      // With many input channels a 1x1 layer is as much the matrix cores' as
      // the memory's: N = 32, 28 x 28, 512 -> 512 runs at 710 TFLOP/s
      // (18.5 us where its bytes alone would stream in 10).
      const double flops = 2.0 * pointwise.batch * pointwise.pixels *
                           pointwise.groups * pointwise.inChansPerGroup *
                           pointwise.outChansPerGroup;
      e.computeUs = std::max(e.computeUs, poplin::kLaunchUs + flops / 7.0e8);
      spread(e, mxk::pointwiseLaunchShape(pointwise, gfx950::numCUs).workgroups,
             1);
      break;
    }
    // (the streaming kernel's K split: the fp32 partial tiles' way out and
    // in again and the second kernel, see splitPenaltyUs)
    const double kSplitUs =
        igemm.splitK > 1 && !igemm.patch
            ? poplin::splitPenaltyUs(mxk::igemmWorkspaceBytes(igemm))
            : 0.0;
    e.reductionUs = kSplitUs;
    e.reductionBytes = kSplitUs > 0 ? mxk::igemmWorkspaceBytes(igemm) : 0;
    bool weighed = false;
    for (const auto &c : candidates)
      if (c.chosen) {
        e.computeUs = c.estimateUs - kSplitUs, weighed = true;
        spread(e, c.workgroups, c.perCU);
      }
    if (weighed)
      break;
    const auto &g = igemm;
    const std::size_t m = std::size_t(g.batch) * g.outD * g.outH * g.outW;
    const std::size_t tiles = (m + 127) / 128 * (coPadded / g.blockN) *
                              g.groups * g.splitK;
    const std::size_t steps =
        (kPadded / g.blockK + g.splitK - 1) / g.splitK;
    const std::size_t perCU = g.blockN == 64 || g.stages == 2 ? 2 : 1;
    double us = poplin::estimateStreaming(tiles, steps, perCU, g.blockN,
                                          g.splitK,
                                          mxk::igemmWorkspaceBytes(igemm));
    // No kernel is faster than its tensors stream.
    us = std::max(us, streamed(inputBytes() + outputBytes() +
                               weightPackedBytes()));
    e.computeUs = us - kSplitUs;
    spread(e, tiles, perCU);
    break;
  }
  }
  if (paddedInputChans) { // the zero-filling copy of the input
    e.rearrangementUs += streamed(2 * inputBytes());
    e.rearrangementBytes += workspaceBytes - paddedInputOffset;
  }
  if (outputPadded) // the fill of the output before the kernel
    e.rearrangementUs += streamed(outputBytes());
  return e;
}

double mxconv_plan::estimatedMicroseconds() const {
  const DetailedEstimate e = detailedEstimate();
  return e.known ? e.totalUs() : -1.0;
}

std::string mxconv_plan::describe() const {
  std::ostringstream os;
  os << "  Plan (gfx950: " << gfx950::numCUs << " CUs, "
     << gfx950::ldsBytesPerCU / 1024 << " KB LDS/CU, wave"
     << gfx950::wavefrontSize << "):\n";
  os << "        kernel                     ";
  switch (kernel) {
  case Kernel::GENERIC:
    os << "generic direct (vector ALU, any parameters)";
    break;
  case Kernel::IGEMM:
    os << "implicit GEMM (MFMA, "
       << (params.inputType == poplar::QUARTER ? "fp8"
           : params.inputType == poplar::FLOAT ? "fp32"
                                               : "fp16")
       << " operands, fp32 accumulate)"
       << (pointwiseOn ? ", pointwise streaming variant" : "")
       << (thinInputOn ? ", kernel rows as k-steps" : "")
       << (igemm.patch ? ", input patch resident in LDS" : "");
    break;
  case Kernel::DEPTHWISE:
    os << (mxk::depthwiseDirectInBlocks(depthwise)
               ? "depthwise direct (vector ALU, one thread per 2x2 block of "
                 "outputs, dilated input)"
           : depthwise.inDilH != 1 || depthwise.inDilW != 1
               ? "depthwise direct (vector ALU, one thread per output "
                 "vector, dilated input)"
           : depthwise.dense3x3 == 2
               ? "depthwise direct (vector ALU, input rows streamed through "
                 "an LDS ring by persistent workgroups)"
           : depthwise.dense3x3
               ? "depthwise direct (vector ALU, dense row loads, small "
                 "workgroups)"
               : "depthwise direct (vector ALU, LDS halo tiles)");
    break;
  }
  os << "\n        reason                     " << reason << "\n";
  os << "        zeroConv                   " << (zeroConv ? "true" : "false")
     << "\n";
  os << "        partialsType               float\n";
  if (wuGroupsPerGroup > 1)
    os << "        conv groups per group      " << wuGroupsPerGroup
       << " (the weight update pass of the layer with that many of its "
       << canonical.numConvGroups * wuGroupsPerGroup
       << " groups taken as one; the diagonal blocks of the fused layer's "
          "deltas are handed back)\n";
  if (kernel == Kernel::IGEMM && thinInputOn) {
    const auto &t = thinInput;
    const mxk::ThinInputLaunch l =
        mxk::thinInputLaunchShape(t, gfx950::numCUs);
    const unsigned steps = mxk::thinInputKSteps(t);
    const unsigned perRow = (t.kW * t.inChans + 7) / 8;
    os << "        gemm M x N x K             "
       << std::size_t(t.batch) * t.outH * t.outW << " x " << t.outChans
       << " x " << steps * 32 << " (a kernel row's " << t.kW << " x "
       << t.inChans << " = " << t.kW * t.inChans
       << " neighbouring elements as " << perRow
       << " chunk(s) of 8; the " << t.kH * perRow << " chunks of " << t.kH
       << " kernel rows in " << steps << " k-step(s) of four)\n";
    os << "        block M x N x K            16 x " << t.outChans
       << " x 32 per wave; tiles of " << l.tileRows
       << " output rows of one image, their input rows in " << l.ldsBytes
       << " bytes of LDS\n";
    os << "        workgroups                 " << l.workgroups
       << " persistent (4 waves) taking " << l.tiles << " tiles in turn on "
       << gfx950::numCUs << " CUs\n";
    os << "        packed weights             [" << t.outChans / 16
       << " blocks of 16][" << steps << " k-steps][64 lanes][8]\n";
  } else if (kernel == Kernel::IGEMM) {
    const auto &g = igemm;
    const std::size_t m = std::size_t(g.batch) * g.outD * g.outH * g.outW;
    const std::size_t k =
        std::size_t(g.kD) * g.kH * g.kW * g.inChansPerGroup;
    const std::size_t tiles = (m + g.blockM - 1) / g.blockM *
                              (coPadded / g.blockN) * g.groups;
    os << "        gemm M x N x K             " << m << " x "
       << g.outChansPerGroup << " x " << k << " (x " << g.groups
       << " groups)\n";
    if (convGroupsPerGroup > 1)
      os << "        conv groups per group      " << convGroupsPerGroup
         << " (" << canonical.numConvGroups << " groups of "
         << canonical.inputChannelsPerConvGroup << " -> "
         << canonical.outputChannelsPerConvGroup << " channels run as "
         << g.groups << " of " << g.inChansPerGroup << " -> "
         << g.outChansPerGroup << ", weights block-diagonal)\n";
    if (pointwiseOn) {
      const std::size_t nTiles = (g.outChansPerGroup + 63) / 64;
      const mxk::PointwiseLaunch l =
          mxk::pointwiseLaunchShape(pointwise, gfx950::numCUs);
      os << "        block M x N x K            " << l.tilePixels
         << " x " << l.chansPerWorkgroup << " x " << k << "\n";
      os << "        workgroups                 " << l.workgroups << " on "
         << gfx950::numCUs << " CUs, each taking " << l.tilesPerWorkgroup
         << " tiles in turn through a ring of " << l.ring
         << " LDS buffers filled by " << l.loaderWaves << " loader waves\n";
      os << "        packed weights             [G=" << g.groups << "]["
         << nTiles * 2 << " blocks of 32][" << k / 16
         << " slices of 16][64 lanes][8]\n";
    } else {
      os << "        block M x N x K            " << g.blockM << " x "
         << g.blockN << " x " << g.blockK << "\n";
      os << "        workgroups                 " << tiles * g.splitK
         << " on " << gfx950::numCUs << " CUs ("
         << std::min<std::size_t>(tiles * g.splitK, gfx950::numCUs)
         << " busy, "
         << (tiles * g.splitK + gfx950::numCUs - 1) / gfx950::numCUs
         << " round(s) of tiles)\n";
      if (g.patch)
        os << "        data path                  input rows of the tile "
              "resident in LDS, weights straight to registers; 8 waves, one "
              "workgroup per CU; MFMA blocks of "
           << (g.patch == 2
                   ? "16 pixels, k-steps taken in turn by the two waves of a "
                     "SIMD\n"
                   : "32 pixels, each k-step halved between the two waves of "
                     "a SIMD\n");
      else if (g.blockN == 128)
        os << "        LDS stages                 " << g.stages
           << (g.stages == 2 ? " (two workgroups per CU)\n"
                             : " (one workgroup per CU)\n");
      if (g.splitK > 1)
        os << "        K split into parts         " << g.splitK
           << " (fp32 partial tiles, summed by a second kernel)\n";
      if (mxk::igemmTapAddressing(g) == mxk::kRangeTaps)
        os << "        tap addressing             ranges of valid kernel rows "
              "and columns (more than 32 taps)\n";
      else if (!igemmPhases.empty())
        os << "        dilated input              " << igemmPhases.size()
           << " phases, one convolution of the undilated input each, in "
              "one launch\n";
      else if (mxk::igemmTapAddressing(g) == mxk::kDilatedTaps)
        os << "        tap addressing             arithmetic (dilated "
              "input)\n";
      if (g.patch)
        os << "        packed weights             [G=" << g.groups << "]["
           << coPadded / 32 << " blocks of 32][" << k * params.inputType.size() / 128
           << " k-steps]"
           << (g.patch == 2 ? "[4 operands]" : "[2 halves][2]")
           << "[64 lanes][16 bytes]\n";
      else
        os << "        packed weights             [G=" << g.groups << "]["
           << coPadded << "][" << kPadded << "]\n";
      if (!candidates.empty()) {
        os << "        tilings weighed            workgroups  per CU  rounds  "
              "k-steps  estimate\n";
        for (const auto &c : candidates) {
          char line[160];
          std::snprintf(line, sizeof line,
                        "          %c %-34s %8zu  %6zu  %6.2f  %7zu  %7.1f us\n",
                        c.chosen ? '*' : ' ', c.name.c_str(), c.workgroups,
                        c.perCU, c.rounds, c.kSteps, c.estimateUs);
          os << line;
        }
      }
      if (paddedInputChans)
        os << "        input channels padded      "
           << params.inputChannelsPerConvGroup << " -> " << paddedInputChans
           << " per group (zero-filled copy in the workspace, every "
              "launch)\n";
    }
  } else if (kernel == Kernel::DEPTHWISE) {
    const auto &d = depthwise;
    os << "        channels                   " << d.channels << "\n";
    if (!d.dense3x3)
      os << "        output tile H x W          " << d.tileH << " x "
         << d.tileW
         << (d.stripPixels == 7
                 ? ", a strip of 7 neighbouring pixels per thread"
                 : d.stripPixels == 4
                       ? ", a strip of 4 neighbouring pixels per thread"
                       : "")
         << "\n";
    if (d.dense3x3 == 2) {
      const mxk::DepthwiseRowsLaunch l = mxk::depthwiseRowsLaunchShape(d);
      os << "        workgroups                 " << l.workgroups << " on "
         << d.cus << " CUs: per image " << l.strips << " strips of "
         << l.colsOut << " output columns x " << l.bands << " bands of "
         << l.rowsOut << " output rows; ring of " << l.ringRows
         << " input rows in LDS filled by " << l.loaderWaves
         << " loader waves, read by " << l.computeWaves << " compute waves\n";
    }
    os << "        packed weights             [" << d.kH * d.kW << "]["
       << d.channels << "]\n";
  } else {
    os << "        packed weights             [G][K][Ci][Co]\n";
  }
  if (depthwiseWeightUpdate) {
    os << "        as a weight update pass    depthwise weight-delta kernel "
          "on the layer's own tensors";
    if (depthwiseForward.dense3x3 == 2) {
      const mxk::DepthwiseRowsLaunch l =
          mxk::depthwiseRowsDeltaLaunchShape(depthwiseForward);
      os << ", rows of both streamed through LDS rings by " << l.workgroups
         << " persistent workgroups (" << l.strips << " strips x " << l.bands
         << " bands of " << l.rowsOut << " rows per image)";
    }
    os << "\n";
  }
  if (denseWeightUpdate) {
    const auto &f = denseForward;
    const std::size_t m = std::size_t(f.batch) * f.outH * f.outW;
    const std::size_t chunks = (m + f.chunkPixels - 1) / f.chunkPixels;
    const std::size_t tiles = std::size_t(f.groups) * f.kH * f.kW *
                              ((f.ci + 127) / 128) * ((f.co + 127) / 128);
    os << "        as a weight update pass    matrix-core weight-delta kernel "
          "on the layer's own tensors (transposing LDS reads): "
       << tiles << " tap x channel tiles x " << chunks << " chunks of "
       << f.chunkPixels << " pixels = " << tiles * chunks
       << " workgroups, fp32 partial tiles summed in order\n";
  }
  if (weightUpdateProduct) {
    const auto &q = weightUpdateProduct->params;
    std::string tiling;
    for (const auto &c : weightUpdateProduct->candidates)
      if (c.chosen)
        tiling = c.name;
    os << "        as a weight update pass    one matrix product, "
          "transpose(deltas) x activations: "
       << q.batchSize << " x " << q.inputChannelsPerConvGroup << " x "
       << q.outputChannelsPerConvGroup
       << " (output channels x batch x input channels), its result in "
          "weight order as it is"
       << (tiling.empty() ? "" : "; " + tiling) << "\n";
  }
  os << "        workspaceBytes             " << workspaceBytes << "\n";
  return os.str();
}

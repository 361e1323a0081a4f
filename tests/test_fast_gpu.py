"""GPU parity of the matrix-core (implicit GEMM) and depthwise kernels against
the CPU oracle, through the C ABI.

Tolerances (relative L2 error against the double-precision oracle fed the same
rounded inputs): fp16 in / fp32 accumulate <= 1e-3; fp8 in / fp32 accumulate
<= 3e-2; +-1 data with fp32 output: exact.  The benchmark configurations are
run at full size and checked on a subset of batch images (the convolution is
independent per image) plus size-independent properties."""
import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, rel_l2

pytestmark = pytest.mark.gpu


def _plan_kernel(plan):
    text = plan.describe()
    for name in ("implicit GEMM", "depthwise direct", "generic direct"):
        if name in text:
            return name
    raise AssertionError(text)


def _run(oracle, p, seed, tol, expect_kernel, dist="normal", bias=True,
         wscale=None, options=None):
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, seed, dist)
    if wscale is not None:
        weights = weights * wscale
    aq, ad = quantize(acts, p.inputType)
    wq, wd = quantize(weights, p.inputType)
    bq, bd = quantize(biases, p.outputType)
    got, plan = run_conv(p, aq, wq, bq if bias else None, options,
                         return_plan=True)
    assert _plan_kernel(plan) == expect_kernel, plan.describe()
    want = oracle.convolution(p, ad, wd, bd if bias else None, threads=8)
    assert got.shape == want.shape
    if tol == 0:
        np.testing.assert_array_equal(got, want)
    else:
        err = rel_l2(got, want)
        assert err <= tol, (err, p)
    return got


IGEMM_CASES = [
    # benchmark config 2 shape (3x3 s1 p1, 128->128, 28x28), reduced batch
    dict(batch=2, field=(28, 28), kernel=(3, 3), ci=128, co=128, pad=1),
    # benchmark config 3 shape (1x1, 256->64, 56x56), reduced batch
    dict(batch=1, field=(56, 56), kernel=(1, 1), ci=256, co=64),
    # M, N, K all ragged against the 128 x {64,128} x 64 tile
    dict(batch=3, field=(9, 7), kernel=(3, 3), ci=8, co=40, pad=1),
    dict(batch=1, field=(5, 5), kernel=(2, 3), ci=24, co=130,
         padLower=(1, 0), padUpper=(0, 2)),
    # stride, kernel dilation, groups
    dict(batch=2, field=(17, 15), kernel=(3, 3), ci=16, co=24, groups=3,
         stride=(2, 1), kdil=(1, 2), pad=2),
    # 1-D field and a tall kernel
    dict(batch=2, field=(50,), kernel=(7,), ci=32, co=16, stride=3, pad=3),
    # truncation folded into the window: input and output truncation
    dict(batch=1, field=(12, 12), kernel=(3, 3), ci=8, co=8, itl=(1, 0),
         itu=(0, 2), otl=(1, 1), otu=(0, 1), pad=1),
    # 0-D field = plain matrix product
    dict(batch=70, field=(), kernel=(), ci=64, co=96),
]


@pytest.mark.parametrize("kw", IGEMM_CASES)
def test_igemm_fp16_matches_oracle(oracle, kw):
    p = make_params(pa.HALF, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 1, 1e-3, "implicit GEMM", wscale=0.1)


@pytest.mark.parametrize("kw", IGEMM_CASES[2:6])
def test_igemm_fp16_in_fp32_out_pm1_exact(oracle, kw):
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 2, 0, "implicit GEMM", dist="pm1")


def test_igemm_blockN_override_and_amp_method(oracle):
    p = make_params(pa.HALF, batch=1, field=(10, 10), kernel=(3, 3), ci=16,
                    co=32, pad=1)
    opts = {"planConstraints":
            '{"method": {"type": "AMP"}, "gfx950": {"blockN": 128}}'}
    _run(oracle, p, 3, 1e-3, "implicit GEMM", options=opts, wscale=0.1)


# 1x1, stride 1, unpadded, 64 / 128 / 256 / 512 input channels per group: the
# streaming kernel of small workgroups.  Ragged pixel counts and channel
# counts against its 64 x 64 tile, groups, 0-D to 2-D fields.
POINTWISE_CASES = [
    dict(batch=2, field=(56, 56), kernel=(1, 1), ci=256, co=64),
    dict(batch=3, field=(7, 11), kernel=(1, 1), ci=128, co=40),
    dict(batch=1, field=(5, 9), kernel=(1, 1), ci=512, co=136, groups=2),
    dict(batch=70, field=(), kernel=(), ci=128, co=96),
    dict(batch=2, field=(33,), kernel=(1,), ci=256, co=8),
    # 64 channels: rows of 128 bytes (the backward pass of a 256 -> 64 layer)
    dict(batch=2, field=(28, 29), kernel=(1, 1), ci=64, co=256),
    dict(batch=3, field=(7, 11), kernel=(1, 1), ci=64, co=72, groups=3),
]


@pytest.mark.parametrize("kw", POINTWISE_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_pointwise_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    plan = pa.Plan(p)
    assert "pointwise streaming variant" in plan.describe(), plan.describe()
    _run(oracle, p, 8, 1e-3, "implicit GEMM", wscale=0.1)


# Several 64-channel tiles of the output per workgroup (the planner's choice
# for large layers that widen the channels), forced onto small ones: pixels
# ragged against the tile, channels that fill the last tile partly, groups.
CHAN_TILE_CASES = [
    (dict(batch=2, field=(28, 29), kernel=(1, 1), ci=64, co=256), 4),
    (dict(batch=2, field=(28, 29), kernel=(1, 1), ci=64, co=256), 2),
    (dict(batch=3, field=(7, 11), kernel=(1, 1), ci=64, co=168), 3),
    (dict(batch=1, field=(19, 9), kernel=(1, 1), ci=64, co=200, groups=2), 4),
    (dict(batch=3, field=(13, 11), kernel=(1, 1), ci=128, co=256), 2),
    (dict(batch=2, field=(9, 31), kernel=(1, 1), ci=128, co=104, groups=3), 2),
    (dict(batch=2, field=(17, 12), kernel=(1, 1), ci=256, co=128), 2),
    (dict(batch=1, field=(6, 40), kernel=(1, 1), ci=256, co=72, groups=2), 2),
]


@pytest.mark.parametrize("kw,tiles", CHAN_TILE_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
@pytest.mark.parametrize("bias", [False, True])
def test_pointwise_channel_tiles_match_oracle(oracle, kw, tiles, out_type,
                                              bias):
    p = make_params(pa.HALF, out_type, **kw)
    options = {"planConstraints": '{"gfx950": {"chanTiles": %d}}' % tiles}
    text = pa.Plan(p, options).describe()
    assert "pointwise streaming variant" in text, text
    assert " x %d x %d\n" % (64 * tiles, kw["ci"]) in text, text
    _run(oracle, p, 14, 1e-3, "implicit GEMM", wscale=0.1, options=options,
         bias=bias)


def test_pointwise_channel_tiles_pm1_exact_and_plan_choice(oracle):
    kw, tiles = CHAN_TILE_CASES[0]
    options = {"planConstraints": '{"gfx950": {"chanTiles": %d}}' % tiles}
    for out_type in (pa.HALF, pa.FLOAT):
        p = make_params(pa.HALF, out_type, **kw)
        _run(oracle, p, 15, 0, "implicit GEMM", dist="pm1", options=options)
    # the planner's own choice: large layers that widen the channels
    def block(**kw):
        import re
        text = pa.Plan(make_params(pa.HALF, **kw)).describe()
        return re.search(r"block M x N x K +(.*)", text).group(1)
    big = dict(batch=32, field=(56, 56), kernel=(1, 1))
    assert block(ci=64, co=256, **big) == "128 x 256 x 64"
    assert block(ci=64, co=192, **big) == "128 x 192 x 64"
    assert block(ci=128, co=256, **big) == "128 x 128 x 128"
    assert block(ci=256, co=128, **big) == "64 x 128 x 256"
    assert block(ci=256, co=64, **big) == "64 x 64 x 256"
    # few pixel tiles per workgroup: one channel tile each
    assert block(ci=128, co=512, batch=32, field=(28, 28),
                 kernel=(1, 1)) == "128 x 64 x 128"
    assert block(**kw) == "128 x 64 x 64"
    # tiles that do not divide the layer's, or too many for the registers
    for bad_kw, bad in ((dict(ci=64, co=192), 2), (dict(ci=128, co=256), 4),
                        (dict(ci=512, co=128), 2)):
        with pytest.raises(pa.MxconvError):
            pa.Plan(make_params(pa.HALF, **bad_kw, **big),
                    {"planConstraints":
                     '{"gfx950": {"chanTiles": %d}}' % bad})


# Input channels that are no power of two, or fewer than 64: the kernel runs
# them as rows of the next size up (16, 32, 64, 128, 256, 512), the chunks
# past the layer's channels loaded from beyond the buffer - zeros - and the
# packed weights zero there.  MobileNet's thin layers and their neighbours:
# pixels ragged against the tile, groups, output channels that fill the last
# tile partly.
THIN_POINTWISE_CASES = [
    dict(batch=2, field=(28, 29), kernel=(1, 1), ci=8, co=48),
    dict(batch=3, field=(17, 9), kernel=(1, 1), ci=16, co=96),
    dict(batch=2, field=(13, 22), kernel=(1, 1), ci=24, co=144),
    dict(batch=1, field=(31, 19), kernel=(1, 1), ci=32, co=16),
    dict(batch=2, field=(9, 14), kernel=(1, 1), ci=40, co=72, groups=2),
    dict(batch=2, field=(12, 12), kernel=(1, 1), ci=96, co=24),
    dict(batch=3, field=(7, 11), kernel=(1, 1), ci=144, co=32),
    dict(batch=1, field=(15, 15), kernel=(1, 1), ci=192, co=64, groups=2),
    dict(batch=2, field=(7, 7), kernel=(1, 1), ci=320, co=1280),
    dict(batch=2, field=(8, 5), kernel=(1, 1), ci=384, co=96),
    dict(batch=1, field=(5, 6), kernel=(1, 1), ci=504, co=40),
]
FORCE_POINTWISE = {"planConstraints": '{"gfx950": {"pointwise": 1}}'}


@pytest.mark.parametrize("kw", THIN_POINTWISE_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_pointwise_any_multiple_of_eight_channels(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    text = pa.Plan(p, FORCE_POINTWISE).describe()
    assert "pointwise streaming variant" in text, text
    # +-1 data: exact, whatever the padding multiplies
    _run(oracle, p, 21, 0 if out_type == pa.FLOAT else 1e-3, "implicit GEMM",
         dist="pm1" if out_type == pa.FLOAT else "normal",
         options=FORCE_POINTWISE, bias=bool(kw["ci"] % 16),
         **({} if out_type == pa.FLOAT else {"wscale": 0.1}))


# fp8 inputs through the same kernel: rows of 16 to 1024 channels (the bytes
# of 8 to 512 fp16 ones), the four pairs of formats, several channel tiles
# per workgroup, groups, bias (which enters the sums divided by the scale).
FP8_POINTWISE_CASES = [
    dict(batch=2, field=(28, 29), kernel=(1, 1), ci=16, co=48),
    dict(batch=3, field=(17, 9), kernel=(1, 1), ci=48, co=96),
    dict(batch=2, field=(13, 22), kernel=(1, 1), ci=128, co=256),
    dict(batch=2, field=(9, 14), kernel=(1, 1), ci=80, co=72, groups=2),
    dict(batch=3, field=(7, 11), kernel=(1, 1), ci=256, co=64),
    dict(batch=1, field=(15, 15), kernel=(1, 1), ci=512, co=128, groups=2),
    dict(batch=2, field=(7, 7), kernel=(1, 1), ci=1024, co=256),
    dict(batch=2, field=(8, 5), kernel=(1, 1), ci=592, co=40),
]


@pytest.mark.parametrize("kw", FP8_POINTWISE_CASES)
@pytest.mark.parametrize("fmt_a,fmt_w", [(1, 1), (1, 0), (0, 1), (0, 0)])
def test_pointwise_fp8_matches_oracle(oracle, kw, fmt_a, fmt_w):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.QUARTER, pa.HALF, **kw)
    print("case", p, fmt_a, fmt_w, flush=True)
    acts, weights, biases = random_data(p, 23, "normal")
    fan_in = p.inputChannelsPerConvGroup
    weights = weights * np.sqrt(2.0 / fan_in)

    def scale_for(x, fmt):
        maxv = 448.0 if fmt == oracle.E4M3 else 57344.0
        return int(np.ceil(np.log2(np.abs(x).max() / maxv)))

    sa, sw = scale_for(acts, fmt_a), scale_for(weights, fmt_w)
    aq, ad = quantize(acts, pa.QUARTER, oracle, fmt_a, sa)
    wq, wd = quantize(weights, pa.QUARTER, oracle, fmt_w, sw)
    bq, bd = quantize(biases, pa.HALF)
    got, plan = run_conv(p, aq, wq, bq, FORCE_POINTWISE,
                         in_meta=pa.quarter_metadata(fmt_a, sa),
                         w_meta=pa.quarter_metadata(fmt_w, sw),
                         return_plan=True)
    assert "pointwise streaming variant" in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    err = rel_l2(got, want)
    assert err <= 1e-3, err


def test_pointwise_fp8_equals_the_big_tile(oracle):
    """The same sums in fp32 from the same fp8 operands: the streaming kernel
    and the big tile agree to the last bit of the half output but for the
    order of the additions (a few results in a thousand differ by one ulp)."""
    from test_fast_gpu import _fp8_case as case
    p = make_params(pa.QUARTER, pa.HALF, batch=2, field=(14, 14),
                    kernel=(1, 1), ci=256, co=128)
    small, _, plan = case(oracle, p, 24, 1, 0)
    assert "pointwise streaming variant" in plan.describe()
    big, want, plan = case(oracle, p, 24, 1, 0, options={
        "planConstraints": '{"gfx950": {"pointwise": 0}}'})
    assert "pointwise streaming variant" not in plan.describe()
    assert rel_l2(small, want) <= 1e-3 and rel_l2(big, want) <= 1e-3
    assert np.mean(small != big) < 0.01


def test_pointwise_pm1_exact_and_big_tile_on_request(oracle):
    p = make_params(pa.HALF, pa.FLOAT, **POINTWISE_CASES[1])
    _run(oracle, p, 9, 0, "implicit GEMM", dist="pm1")
    opts = {"planConstraints": '{"gfx950": {"kernel": "igemm"}}'}
    assert "pointwise" not in pa.Plan(p, opts).describe()
    _run(oracle, p, 9, 0, "implicit GEMM", dist="pm1", options=opts)


DW_CASES = [
    # benchmark config 4 shape (3x3 s2 p1, C=96, 112x112), reduced batch
    dict(batch=2, field=(112, 112), kernel=(3, 3), groups=96, stride=2, pad=1),
    dict(batch=3, field=(9, 11), kernel=(3, 3), groups=8, pad=1),
    dict(batch=1, field=(13, 7), kernel=(5, 2), groups=24, stride=(1, 2),
         kdil=(2, 1), padLower=(3, 0), padUpper=(1, 1)),
    dict(batch=2, field=(31,), kernel=(4,), groups=16, stride=2, pad=2),
]


@pytest.mark.parametrize("kw", DW_CASES)
def test_depthwise_fp16_matches_oracle(oracle, kw):
    p = make_params(pa.HALF, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 4, 1e-3, "depthwise direct")


# 3x3, dilation 1, stride 1 or 2: the kernel built from small dense-loading
# workgroups.  Shapes chosen so that workgroup blocks are ragged in both
# directions, channel vectors per pixel vary (1 .. 28), padding is asymmetric,
# negative (truncation) or absent, and images are narrower than one block.
DW3X3_CASES = [
    dict(batch=2, field=(23, 45), kernel=(3, 3), groups=96, stride=2, pad=1),
    dict(batch=2, field=(23, 45), kernel=(3, 3), groups=96, stride=1, pad=1),
    dict(batch=1, field=(8, 70), kernel=(3, 3), groups=8, stride=1),
    dict(batch=3, field=(7, 5), kernel=(3, 3), groups=224, stride=2,
         padLower=(2, 0), padUpper=(0, 3)),
    dict(batch=2, field=(16, 19), kernel=(3, 3), groups=40, stride=2,
         itl=(1, 2), itu=(2, 0), otl=(1, 0), otu=(0, 1), pad=1),
    dict(batch=1, field=(3, 3), kernel=(3, 3), groups=16, stride=1),
    dict(batch=5, field=(33, 64), kernel=(3, 3), groups=32, stride=2, pad=1),
]


@pytest.mark.parametrize("kw", DW3X3_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_depthwise_3x3_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    from gpu_helpers import run_conv  # noqa: F401  (GPU needed from here on)
    got = _run(oracle, p, 6, 1e-3, "depthwise direct")
    assert got.size


def test_depthwise_3x3_plan_reports_its_kernel_and_tile_override(oracle):
    p = make_params(pa.HALF, **DW3X3_CASES[0])
    plan = pa.Plan(p)
    assert "dense row loads" in plan.describe(), \
        plan.describe()
    opts = {"planConstraints": '{"gfx950": {"tileH": 2, "tileW": 5}}'}
    tiled = pa.Plan(p, opts)
    assert "LDS halo tiles" in tiled.describe(), tiled.describe()
    # the LDS-tiled kernel still serves the same shape when asked to
    _run(oracle, p, 7, 1e-3, "depthwise direct", options=opts)


ROW_RING = {"planConstraints": '{"gfx950": {"rowRing": 1}}'}
RING = "input rows streamed through an LDS ring"


# The persistent kernel with a ring of input rows in LDS, forced onto the same
# shapes (the planner keeps it for layers that fill the chip): bands of one
# row, strips narrower than the image and wider, images smaller than a ring.
@pytest.mark.parametrize("kw", DW3X3_CASES + [
    # several strips (28 channel vectors per pixel: 13 output columns each)
    # and bands of more than one row
    dict(batch=48, field=(40, 60), kernel=(3, 3), groups=224, stride=2,
         pad=1),
    # stride 1, rows longer than a strip
    dict(batch=40, field=(30, 150), kernel=(3, 3), groups=64, stride=1,
         pad=1),
    # more channels than the small-workgroup kernel takes: strips of a few
    # columns, eight and six compute waves
    dict(batch=6, field=(20, 37), kernel=(3, 3), groups=256, stride=1, pad=1),
    dict(batch=5, field=(14, 14), kernel=(3, 3), groups=576, stride=2, pad=1),
    dict(batch=3, field=(7, 7), kernel=(3, 3), groups=960, stride=1, pad=1),
    # the most the kernel takes: one output column per strip
    dict(batch=2, field=(6, 5), kernel=(3, 3), groups=2048, stride=1, pad=1),
    dict(batch=2, field=(9, 7), kernel=(3, 3), groups=2048, stride=2, pad=1),
    # 5 x 5 taps: both strides, strips and bands ragged, more padding on one
    # side than the other, wide pixels
    dict(batch=9, field=(28, 28), kernel=(5, 5), groups=240, stride=1, pad=2),
    dict(batch=7, field=(31, 45), kernel=(5, 5), groups=144, stride=2, pad=2),
    dict(batch=3, field=(14, 14), kernel=(5, 5), groups=672, stride=1,
         padLower=(2, 1), padUpper=(3, 2)),
    dict(batch=2, field=(11, 9), kernel=(5, 5), groups=1152, stride=2, pad=2),
    dict(batch=40, field=(20, 70), kernel=(5, 5), groups=16, stride=1, pad=2),
])
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_depthwise_row_ring_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    assert RING in pa.Plan(p, ROW_RING).describe()
    _run(oracle, p, 8, 1e-3, "depthwise direct", options=ROW_RING)


def test_depthwise_row_ring_pm1_exact(oracle):
    for kw in (DW3X3_CASES[0], DW3X3_CASES[3], DW3X3_CASES[6]):
        p = make_params(pa.HALF, pa.FLOAT, **kw)
        _run(oracle, p, 9, 0, "depthwise direct", dist="pm1",
             options=ROW_RING)


def test_depthwise_row_ring_plan_choice():
    big = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                      groups=96, stride=2, pad=1)
    text = pa.Plan(big).describe()
    assert RING in text, text
    assert ("256 on 256 CUs: per image 2 strips of 28 output columns x 4 "
            "bands of 14 output rows") in text, text
    off = pa.Plan(big, {"planConstraints": '{"gfx950": {"rowRing": 0}}'})
    assert "dense row loads" in off.describe()
    assert "read by 6 compute waves" in text, text
    # stride 1: eight compute waves take wider strips
    s1 = make_params(pa.HALF, batch=32, field=(56, 56), kernel=(3, 3),
                     groups=144, stride=1, pad=1)
    text = pa.Plan(s1).describe()
    assert ("256 on 256 CUs: per image 2 strips of 28 output columns x 4 "
            "bands of 14 output rows") in text, text
    assert "read by 8 compute waves" in text, text
    # few rows per CU: the small workgroups stay
    small = make_params(pa.HALF, **DW3X3_CASES[0])
    assert "dense row loads" in pa.Plan(small).describe()
    # ... unless the layer has more channels than they take (224)
    wide = make_params(pa.HALF, batch=1, field=(14, 14), kernel=(3, 3),
                       groups=576, stride=1, pad=1)
    assert RING in pa.Plan(wide).describe()
    assert "LDS halo tiles" in pa.Plan(
        wide, {"planConstraints": '{"gfx950": {"rowRing": 0}}'}).describe()
    # 5 x 5 taps take it too where strips are four columns wide or more (and
    # at stride 2 bands six rows long)
    five = dict(batch=32, kernel=(5, 5), pad=2)
    assert RING in pa.Plan(make_params(
        pa.HALF, field=(28, 28), groups=240, **five)).describe()
    assert RING in pa.Plan(make_params(
        pa.HALF, field=(56, 56), groups=144, stride=2, **five)).describe()
    assert "LDS halo tiles" in pa.Plan(make_params(
        pa.HALF, field=(28, 28), groups=240, stride=2, **five)).describe()
    assert "LDS halo tiles" in pa.Plan(make_params(
        pa.HALF, field=(7, 7), groups=1152, **five)).describe()
    # not a 3x3 or 5x5 kernel: the constraint cannot be met
    with pytest.raises(pa.MxconvError):
        pa.Plan(make_params(pa.HALF, batch=2, field=(20, 20), kernel=(7, 7),
                            groups=32, pad=3), ROW_RING)


def test_depthwise_fp32_out_pm1_exact(oracle):
    p = make_params(pa.HALF, pa.FLOAT, **DW_CASES[1])
    _run(oracle, p, 5, 0, "depthwise direct", dist="pm1")


def _fp8_case(oracle, p, seed, fmt_a, fmt_w, options=None):
    """values ~N(0,1) (weights scaled), per-tensor power-of-two scale chosen
    so the largest magnitude lands below the format's maximum."""
    from gpu_helpers import quantize, run_conv
    acts, weights, _ = random_data(p, seed, "normal")
    fan_in = p.inputChannelsPerConvGroup * int(np.prod(p.kernelShape))
    weights = weights * np.sqrt(2.0 / max(fan_in, 1))

    def scale_for(x, fmt):
        maxv = 448.0 if fmt == oracle.E4M3 else 57344.0
        m = np.abs(x).max()
        return int(np.ceil(np.log2(m / maxv))) if m > 0 else 0

    sa, sw = scale_for(acts, fmt_a), scale_for(weights, fmt_w)
    aq, ad = quantize(acts, pa.QUARTER, oracle, fmt_a, sa)
    wq, wd = quantize(weights, pa.QUARTER, oracle, fmt_w, sw)
    got, plan = run_conv(p, aq, wq, None, options,
                         in_meta=pa.quarter_metadata(fmt_a, sa),
                         w_meta=pa.quarter_metadata(fmt_w, sw),
                         return_plan=True)
    want = oracle.convolution(p, ad, wd, threads=8)
    return got, want, plan


@pytest.mark.parametrize("fmt_a,fmt_w", [(1, 1), (1, 0), (0, 1), (0, 0)])
def test_igemm_fp8_matches_oracle(oracle, fmt_a, fmt_w):
    # benchmark config 5 shape (3x3 s1 p1, 256->256, 14x14), reduced batch
    p = make_params(pa.QUARTER, pa.HALF, batch=2, field=(14, 14),
                    kernel=(3, 3), ci=256, co=256, pad=1)
    got, want, plan = _fp8_case(oracle, p, 6, fmt_a, fmt_w)
    assert _plan_kernel(plan) == "implicit GEMM"
    err = rel_l2(got, want)
    assert err <= 3e-2, err
    # the inputs are exact in fp8, so the only error is fp32 accumulation and
    # the fp16 output rounding: far below the fp8 budget
    assert err <= 1e-3, err


def test_igemm_fp8_ragged_shapes(oracle):
    p = make_params(pa.QUARTER, pa.HALF, batch=3, field=(7, 9), kernel=(3, 2),
                    ci=16, co=40, groups=2, stride=(1, 2), pad=1)
    got, want, plan = _fp8_case(oracle, p, 7, 1, 1)
    assert _plan_kernel(plan) == "implicit GEMM"
    assert rel_l2(got, want) <= 1e-3


def test_generic_fp8_matches_oracle(oracle):
    # Ci = 4 is not a whole 16-byte vector: falls back to the generic kernel
    p = make_params(pa.QUARTER, pa.HALF, batch=2, field=(6, 6), kernel=(3, 3),
                    ci=4, co=5, pad=1)
    got, want, plan = _fp8_case(oracle, p, 8, 1, 0)
    assert _plan_kernel(plan) == "generic direct"
    assert rel_l2(got, want) <= 1e-3


def test_quarter_small_integer_data_is_exact(oracle):
    """The reference draws quarter test data as small integers so that they
    are exactly representable (lib/poplibs_test/Util.cpp:140-142); with a
    fp32 accumulate the result is then exact up to the fp16 output."""
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.QUARTER, pa.HALF, batch=1, field=(8, 8), kernel=(3, 3),
                    ci=16, co=16, pad=1)
    g = np.random.default_rng(9)
    acts = g.integers(-3, 4, (1, 16, 8, 8)).astype(np.float64)
    weights = g.integers(-1, 2, (1, 16, 16, 3, 3)).astype(np.float64)
    aq, ad = quantize(acts, pa.QUARTER, oracle, 1, 0)
    wq, wd = quantize(weights, pa.QUARTER, oracle, 1, 0)
    np.testing.assert_array_equal(ad, acts)
    got = run_conv(p, aq, wq, None, None, in_meta=0x80, w_meta=0x80)
    want = oracle.convolution(p, ad, wd)
    assert np.abs(want).max() < 2048  # exactly representable in fp16
    np.testing.assert_array_equal(got, want)
    # metadata scales multiply the result by 2^(sIn + sW)
    got2 = run_conv(p, aq, wq, None, None,
                    in_meta=pa.quarter_metadata(1, 1),
                    w_meta=pa.quarter_metadata(1, 2))
    np.testing.assert_array_equal(got2, want * 8.0)
    got3 = run_conv(p, aq, wq, None, None,
                    in_meta=pa.quarter_metadata(1, -2),
                    w_meta=pa.quarter_metadata(1, -1))
    np.testing.assert_array_equal(got3, want / 8.0)


# ---- benchmark configurations at full size ---------------------------------

def _full_size(oracle, p, seed, tol, kernel, act_fn=None, w_std=1.0,
               images=8, recipe=False):
    """recipe: the benchmark's seeded inputs (poplibs_amd.synthetic:
    mt19937_64(seed) for the activations, seed + 1 for the weights, Box-Muller
    normals in the order of the external arrays) instead of numpy's
    generator, so that the test sees the very tensors bench.py times."""
    from gpu_helpers import quantize, run_conv
    ashape = (p.batchSize, p.getNumInputChans(), *p.inputFieldShape)
    wshape = (p.numConvGroups, p.outputChannelsPerConvGroup,
              p.inputChannelsPerConvGroup, *p.kernelShape)
    if recipe:
        from poplibs_amd import synthetic
        acts = synthetic.normal(seed, ashape)
        weights = synthetic.normal(seed + 1, wshape, w_std)
    else:
        g = np.random.default_rng(seed)
        acts = g.standard_normal(ashape)
        weights = g.standard_normal(wshape) * w_std
    if act_fn:
        acts = act_fn(acts)
    aq, ad = quantize(acts, p.inputType)
    wq, wd = quantize(weights, p.inputType)
    got, plan = run_conv(p, aq, wq, None, None, return_plan=True)
    assert _plan_kernel(plan) == kernel
    # `images` images spread over the batch, first and last included,
    # against the oracle, each to the tolerance
    picked = sorted({round(i * (p.batchSize - 1) / (images - 1))
                     for i in range(images)})
    some = pa.ConvParams.from_c(p.to_c())
    some.batchSize = len(picked)
    want = oracle.convolution(some, ad[picked], wd, threads=8)
    for i, b in enumerate(picked):
        err = rel_l2(got[b], want[i])
        assert err <= tol, (b, err)
    # size-independent property: images are independent, so reversing the
    # batch reverses the output, bit for bit
    got_rev = run_conv(p, aq[::-1].copy(), wq, None, None, plan=plan)
    assert np.array_equal(got_rev, got[::-1])
    return got


def test_baseline_config2_full(oracle):
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    assert p.getFwdFlops() == 7050625024
    _full_size(oracle, p, 0, 1e-3, "implicit GEMM",
               w_std=np.sqrt(2.0 / (9 * 128)))


def test_baseline_config3_full(oracle):
    p = make_params(pa.HALF, batch=32, field=(56, 56), kernel=(1, 1), ci=256,
                    co=64)
    assert p.getFwdFlops() == 3288334336
    _full_size(oracle, p, 0, 1e-3, "implicit GEMM",
               act_fn=lambda x: np.maximum(x, 0), w_std=np.sqrt(2.0 / 256))


def test_baseline_config4_full(oracle):
    p = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                    groups=96, stride=2, pad=1)
    assert p.getFwdFlops() == 171350016
    assert p.getOutputFieldShape() == [56, 56]
    _full_size(oracle, p, 0, 1e-3, "depthwise direct", w_std=np.sqrt(2.0 / 9))


def test_baseline_config5_full(oracle):
    from gpu_helpers import run_conv
    p = make_params(pa.QUARTER, pa.HALF, batch=64, field=(14, 14),
                    kernel=(3, 3), ci=256, co=256, pad=1)
    assert p.getFwdFlops() == 13421772800
    # quantise exactly as the configuration states, check eight images; the
    # oracle receives the dequantised values, so the error measured is that of
    # the accumulation and the fp16 output rounding
    from gpu_helpers import quantize
    g = np.random.default_rng(0)
    acts = g.standard_normal((64, 256, 14, 14))
    weights = g.standard_normal((1, 256, 256, 3, 3)) * np.sqrt(2 / (9 * 256))
    sa = int(np.ceil(np.log2(np.abs(acts).max() / 448.0)))
    sw = int(np.ceil(np.log2(np.abs(weights).max() / 448.0)))
    aq, ad = quantize(acts, pa.QUARTER, oracle, 1, sa)
    wq, wd = quantize(weights, pa.QUARTER, oracle, 1, sw)
    got, plan = run_conv(p, aq, wq, None, None,
                         in_meta=pa.quarter_metadata(1, sa),
                         w_meta=pa.quarter_metadata(1, sw), return_plan=True)
    assert _plan_kernel(plan) == "implicit GEMM"
    picked = [0, 9, 18, 27, 36, 45, 54, 63]
    some = pa.ConvParams.from_c(p.to_c())
    some.batchSize = len(picked)
    want = oracle.convolution(some, ad[picked], wd, threads=8)
    for i, b in enumerate(picked):
        # against the dequantised inputs only accumulation and the fp16
        # output round: well inside the 3e-2 fp8 budget
        err = rel_l2(got[b], want[i])
        assert err <= 3e-2 and err <= 1e-3, (b, err)


# The same four configurations on the benchmark's own seeded inputs (the
# recipe of poplibs_amd/synthetic.py that bench.py draws from, seed 0 for the
# activations and 1 for the weights): tests and benchmark see identical data.

def test_baseline_config2_recipe_inputs(oracle):
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    _full_size(oracle, p, 0, 1e-3, "implicit GEMM",
               w_std=(2 / (9 * 128)) ** .5, recipe=True)


def test_baseline_config3_recipe_inputs(oracle):
    p = make_params(pa.HALF, batch=32, field=(56, 56), kernel=(1, 1), ci=256,
                    co=64)
    _full_size(oracle, p, 0, 1e-3, "implicit GEMM",
               act_fn=lambda x: np.maximum(x, 0), w_std=(2 / 256) ** .5,
               recipe=True)


def test_baseline_config4_recipe_inputs(oracle):
    p = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                    groups=96, stride=2, pad=1)
    _full_size(oracle, p, 0, 1e-3, "depthwise direct", w_std=(2 / 9) ** .5,
               recipe=True)


def test_baseline_config5_recipe_inputs(oracle):
    """configs[4] as bench.py prepares it: normals from the recipe, per-tensor
    power-of-two scales e = ceil(log2(max|x| / 448)), values / 2^e rounded to
    E4M3; eight images against the oracle on the dequantised values."""
    from gpu_helpers import quantize, run_conv
    from poplibs_amd import synthetic
    p = make_params(pa.QUARTER, pa.HALF, batch=64, field=(14, 14),
                    kernel=(3, 3), ci=256, co=256, pad=1)
    acts = synthetic.normal(0, (64, 256, 14, 14))
    weights = synthetic.normal(1, (1, 256, 256, 3, 3), (2 / (9 * 256)) ** .5)
    sa = int(np.ceil(np.log2(np.abs(acts).max() / 448.0)))
    sw = int(np.ceil(np.log2(np.abs(weights).max() / 448.0)))
    aq, ad = quantize(acts, pa.QUARTER, oracle, 1, sa)
    wq, wd = quantize(weights, pa.QUARTER, oracle, 1, sw)
    got, plan = run_conv(p, aq, wq, None, None,
                         in_meta=pa.quarter_metadata(1, sa),
                         w_meta=pa.quarter_metadata(1, sw), return_plan=True)
    assert _plan_kernel(plan) == "implicit GEMM"
    picked = [0, 9, 18, 27, 36, 45, 54, 63]
    some = pa.ConvParams.from_c(p.to_c())
    some.batchSize = len(picked)
    want = oracle.convolution(some, ad[picked], wd, threads=8)
    for i, b in enumerate(picked):
        err = rel_l2(got[b], want[i])
        assert err <= 3e-2 and err <= 1e-3, (b, err)


# Kernels of more than 32 taps (valid-range tap addressing) and dilated
# (zero-stuffed) inputs (arithmetic tap addressing), the shapes weight update
# and backward passes bring.
GENERAL_CASES = [
    # 7x7 = 49 taps; channel block of a whole k-step per tap (uniform) or less
    dict(batch=2, field=(20, 19), kernel=(7, 7), ci=64, co=40, pad=3),
    dict(batch=2, field=(20, 19), kernel=(7, 7), ci=8, co=72, pad=3,
         stride=2),
    # backward pass of a stride-2 3x3 layer: input dilated by 2
    dict(batch=2, field=(14, 15), kernel=(3, 3), ci=64, co=16, idil=2,
         padLower=(1, 1), padUpper=(2, 2)),
    dict(batch=3, field=(7, 9), kernel=(3, 2), ci=16, co=136, idil=(3, 2),
         pad=2, kdil=(1, 2), groups=2),
    # dilation and truncation together, 1-D
    dict(batch=2, field=(33,), kernel=(5,), ci=24, co=8, idil=2, itl=(2,),
         itu=(1,), pad=4, stride=3),
    # a window that strides over a dilated input: arithmetic on every tap
    dict(batch=2, field=(11, 12), kernel=(3, 3), ci=64, co=24, idil=2,
         stride=(2, 3), pad=2),
    # a weight-update-like pass: the "kernel" is a whole 12x12 field, dilated
    dict(batch=16, field=(26, 26), kernel=(12, 12), ci=8, co=24, kdil=2,
         padLower=(1, 1), padUpper=(0, 0)),
    # one dimension, a kernel of more than 255 taps (a 1-D layer's weight
    # update pass): windows that hang over both ends of the field, and a
    # dilated kernel that steps over it
    dict(batch=3, field=(500,), kernel=(300,), ci=8, co=24, pad=40),
    dict(batch=2, field=(1200,), kernel=(397,), ci=16, co=8, kdil=3,
         padLower=(5,), padUpper=(17,), stride=2),
    # (and with rows: 3 x 280)
    dict(batch=2, field=(6, 300), kernel=(3, 280), ci=8, co=16,
         padLower=(1, 3), padUpper=(1, 0)),
]


@pytest.mark.parametrize("kw", GENERAL_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_igemm_general_addressing_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, 5, "normal")
    aq, ad = quantize(acts, pa.HALF)
    wq, wd = quantize(weights * 0.05, pa.HALF)
    got, plan = run_conv(p, aq, wq, return_plan=True)
    assert ("tap addressing" in plan.describe()
            or "phases" in plan.describe()), plan.describe()
    want = oracle.convolution(p, ad, wd, threads=8)
    assert rel_l2(got, want) <= 1e-3, (rel_l2(got, want), plan.describe())


SPLIT_K_CASES = [
    # (params, forced parts or None for the planner's choice)
    (dict(batch=1, field=(6, 6), kernel=(3, 3), ci=512, co=128, pad=1), None),
    (dict(batch=2, field=(9, 7), kernel=(3, 3), ci=64, co=40, pad=1), 3),
    (dict(batch=2, field=(9, 7), kernel=(3, 3), ci=64, co=40, pad=1), 9),
    (dict(batch=2, field=(9, 7), kernel=(3, 3), ci=8, co=136, pad=1,
          groups=2), 2),
    # (72 k-steps: long enough for the parts to pay for their round trip)
    (dict(batch=16, field=(26, 26), kernel=(12, 12), ci=32, co=24, kdil=2,
          padLower=(1, 1), padUpper=(0, 0)), None),
    # channel counts that are no multiple of four: the parts are added one
    # channel per thread
    (dict(batch=2, field=(9, 7), kernel=(3, 3), ci=64, co=3, pad=1), 4),
    (dict(batch=1, field=(8, 8), kernel=(5, 5), ci=96, co=7, pad=2, groups=3),
     None),
]


@pytest.mark.parametrize("kw,parts", SPLIT_K_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_igemm_split_k_matches_oracle(oracle, kw, parts, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, parts, flush=True)
    from gpu_helpers import quantize, run_conv
    options = None
    if parts:
        options = {"planConstraints": '{"gfx950": {"splitK": %d}}' % parts}
    acts, weights, biases = random_data(p, 6, "normal")
    aq, ad = quantize(acts, pa.HALF)
    wq, wd = quantize(weights * 0.05, pa.HALF)
    bq, bd = quantize(biases, out_type)
    got, plan = run_conv(p, aq, wq, bq, options, return_plan=True)
    assert "K split into parts" in plan.describe(), plan.describe()
    if parts:
        assert "K split into parts         %d" % parts in plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert rel_l2(got, want) <= 1e-3, (rel_l2(got, want), plan.describe())


FP32_CASES = [
    # the reference's own CPU-runnable configuration: 3x3, 16 -> 16, 32x32
    dict(batch=1, field=(32, 32), kernel=(3, 3), ci=16, co=16, pad=1),
    # a k-step inside one tap (32 floats of channels) ...
    dict(batch=2, field=(14, 14), kernel=(3, 3), ci=64, co=128, pad=1),
    # ... and k-steps that span taps, ragged against the tile
    dict(batch=3, field=(9, 7), kernel=(3, 3), ci=4, co=40, pad=1),
    dict(batch=1, field=(5, 5), kernel=(2, 3), ci=12, co=130,
         padLower=(1, 0), padUpper=(0, 2)),
    dict(batch=2, field=(17, 15), kernel=(3, 3), ci=8, co=24, groups=3,
         stride=(2, 1), kdil=(1, 2), pad=2),
    # dilated input, many taps, a plain matrix product
    dict(batch=2, field=(6, 5), kernel=(3, 3), ci=8, co=16, idil=(2, 3),
         pad=2),
    dict(batch=1, field=(13, 13), kernel=(7, 7), ci=4, co=8, pad=3),
    dict(batch=70, field=(), kernel=(), ci=96, co=64),
]


@pytest.mark.parametrize("kw", FP32_CASES)
@pytest.mark.parametrize("out_type", [pa.FLOAT, pa.HALF])
def test_igemm_fp32_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.FLOAT, out_type, **kw)
    print("case", p, flush=True)
    # fp32 products and sums: the fp16 output rounding is the only other error
    _run(oracle, p, 21, 2e-6 if out_type == pa.FLOAT else 5e-4,
         "implicit GEMM", wscale=0.1)


def test_igemm_fp32_of_signs_is_exact(oracle):
    p = make_params(pa.FLOAT, pa.FLOAT, batch=2, field=(9, 9), kernel=(3, 3),
                    ci=32, co=72, pad=1)
    _run(oracle, p, 22, 0, "implicit GEMM", dist="pm1")


def test_igemm_fp32_split_k(oracle):
    p = make_params(pa.FLOAT, pa.FLOAT, batch=1, field=(6, 6), kernel=(3, 3),
                    ci=256, co=128, pad=1)
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, 23, "normal")
    aq, ad = quantize(acts, pa.FLOAT)
    wq, wd = quantize(weights * 0.05, pa.FLOAT)
    bq, bd = quantize(biases, pa.FLOAT)
    got, plan = run_conv(p, aq, wq, bq, None, return_plan=True)
    assert "fp32 operands" in plan.describe(), plan.describe()
    assert "K split into parts" in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert rel_l2(got, want) <= 2e-6


PADDED_CHANNEL_CASES = [
    # a first layer: 3 input channels, 7x7 stride 2
    (pa.HALF, dict(batch=2, field=(40, 40), kernel=(7, 7), ci=3, co=64,
                   stride=2, pad=3)),
    # groups, each padded by itself; ragged outputs
    (pa.HALF, dict(batch=4, field=(20, 20), kernel=(3, 3), ci=4, co=12,
                   groups=5, pad=1)),
    (pa.HALF, dict(batch=6, field=(16, 18), kernel=(3, 3), ci=13, co=40,
                   pad=1, stride=(1, 2))),
    (pa.FLOAT, dict(batch=8, field=(24, 24), kernel=(3, 3), ci=3, co=32,
                    pad=1)),
    (pa.FLOAT, dict(batch=2, field=(24, 24), kernel=(3, 3), ci=6, co=16,
                    groups=2, idil=2, pad=2)),
    (pa.QUARTER, dict(batch=4, field=(24, 24), kernel=(3, 3), ci=5, co=32,
                      pad=1)),
]


@pytest.mark.parametrize("in_type,kw", PADDED_CHANNEL_CASES)
def test_igemm_pads_odd_channel_counts(oracle, in_type, kw):
    out_type = pa.FLOAT if in_type == pa.FLOAT else pa.HALF
    p = make_params(in_type, out_type, **kw)
    print("case", p, flush=True)
    if in_type == pa.QUARTER:
        got, want, plan = _fp8_case(oracle, p, 31, 1, 1)
    else:
        from gpu_helpers import quantize, run_conv
        acts, weights, biases = random_data(p, 31, "normal")
        aq, ad = quantize(acts, in_type)
        wq, wd = quantize(weights * 0.1, in_type)
        bq, bd = quantize(biases, out_type)
        # (each group by itself: taken as one, the two groups of six fp32
        # channels are whole vectors and need no padding; and not the kernel
        # that reads up to four half channels as they are)
        got, plan = run_conv(
            p, aq, wq, bq,
            {"planConstraints":
             '{"convGroupsPerGroup": 1, "gfx950": {"thinInput": 0}}'},
            return_plan=True)
        want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert "input channels padded" in plan.describe(), plan.describe()
    assert rel_l2(got, want) <= (2e-6 if in_type == pa.FLOAT else 1e-3)


DEPTH_CASES = [
    # a 3-D UNet style layer
    (pa.HALF, dict(batch=2, field=(6, 10, 9), kernel=(3, 3, 3), ci=16, co=24,
                   pad=1)),
    # stride, padding and kernel dilation different in every dimension
    (pa.HALF, dict(batch=2, field=(9, 8, 11), kernel=(2, 3, 3), ci=8, co=40,
                   stride=(2, 1, 2), kdil=(2, 1, 1), padLower=(1, 0, 2),
                   padUpper=(2, 1, 0), groups=2)),
    (pa.HALF, dict(batch=1, field=(5, 7, 6), kernel=(3, 1, 2), ci=64, co=130,
                   padLower=(2, 0, 1), padUpper=(0, 0, 0))),
    # truncation in depth; few channels (padded)
    (pa.HALF, dict(batch=2, field=(8, 12, 12), kernel=(3, 3, 3), ci=3, co=32,
                   itl=(1, 0, 0), itu=(0, 1, 0), pad=1)),
    (pa.FLOAT, dict(batch=2, field=(5, 6, 7), kernel=(3, 3, 3), ci=8, co=16,
                    pad=1)),
    (pa.QUARTER, dict(batch=2, field=(5, 6, 7), kernel=(3, 3, 3), ci=16,
                      co=16, pad=1)),
    # a depth the window does not slide over: folded into the batch
    (pa.HALF, dict(batch=2, field=(5, 9, 9), kernel=(1, 7, 7), ci=8, co=16,
                   padLower=(0, 3, 3), padUpper=(0, 3, 3))),
    # more than 32 taps in three dimensions: ranges of valid planes, rows and
    # columns (what a weight update pass of a 3-D layer brings)
    (pa.HALF, dict(batch=2, field=(6, 7, 8), kernel=(3, 3, 4), ci=16, co=24,
                   pad=1)),
    (pa.HALF, dict(batch=2, field=(9, 8, 7), kernel=(5, 5, 5), ci=64, co=40,
                   padLower=(2, 1, 3), padUpper=(1, 2, 2), stride=(1, 2, 1),
                   kdil=(2, 1, 1))),
]


@pytest.mark.parametrize("in_type,kw", DEPTH_CASES)
def test_igemm_three_field_dimensions(oracle, in_type, kw):
    out_type = pa.FLOAT if in_type == pa.FLOAT else pa.HALF
    p = make_params(in_type, out_type, **kw)
    print("case", p, flush=True)
    if in_type == pa.QUARTER:
        got, want, plan = _fp8_case(oracle, p, 41, 1, 1)
        assert _plan_kernel(plan) == "implicit GEMM", plan.describe()
        assert rel_l2(got, want) <= 1e-3
    else:
        _run(oracle, p, 41, 2e-6 if in_type == pa.FLOAT else 1e-3,
             "implicit GEMM", wscale=0.1)


def test_igemm_three_dimensions_of_signs_is_exact(oracle):
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(4, 6, 5),
                    kernel=(3, 3, 3), ci=16, co=24, pad=1, stride=(1, 2, 1))
    _run(oracle, p, 42, 0, "implicit GEMM", dist="pm1")


def test_igemm_input_beyond_two_gigabytes(oracle):
    """The input is addressed with 32-bit offsets from the first image a tile
    reads, so the tensor itself may exceed 2^31 bytes: every image of such a
    batch must come out exactly as it does alone."""
    import torch
    from poplibs_amd import capi
    kw = dict(field=(512, 512), kernel=(3, 3), ci=256, co=16, pad=1)
    big = make_params(pa.HALF, pa.HALF, batch=18, **kw)
    one = make_params(pa.HALF, pa.HALF, batch=1, **kw)
    plan_big, plan_one = pa.Plan(big), pa.Plan(one)
    assert _plan_kernel(plan_big) == "implicit GEMM", plan_big.describe()
    assert plan_big.buffer_bytes(capi.BUF_INPUT) > 2 ** 31
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn((18, 512, 512, 256), generator=g, device=dev,
                    dtype=torch.float16)           # channels-last, as documented
    w = (torch.randn((1, 16, 256, 3, 3), generator=g, device=dev,
                     dtype=torch.float16) * 0.02)

    def buf(plan, which):
        return torch.empty(max(plan.buffer_bytes(which), 16),
                           dtype=torch.uint8, device=dev)

    def run(plan, x_part):
        wp, out = buf(plan, capi.BUF_WEIGHTS_PACKED), buf(plan, capi.BUF_OUTPUT)
        ws = buf(plan, capi.BUF_WORKSPACE)
        plan.pack_weights(w.data_ptr(), wp.data_ptr())
        plan.fwd(x_part.data_ptr(), wp.data_ptr(), out.data_ptr(), None,
                 ws.data_ptr(), ws.numel())
        torch.cuda.synchronize()
        return out.view(torch.float16)

    got = run(plan_big, x).view(18, 512, 512, 16)
    for image in (0, 7, 8, 17):
        alone = run(plan_one, x[image].contiguous()).view(512, 512, 16)
        assert torch.equal(got[image], alone), image
    assert torch.isfinite(got).all() and got.abs().max() > 0


def test_depthwise_batch_beyond_one_launch(oracle):
    """A depthwise batch too large for one launch's 32-bit offsets goes out
    in several launches: every image as it comes out alone."""
    import torch
    from poplibs_amd import capi
    kw = dict(field=(112, 112), kernel=(3, 3), groups=96, stride=2, pad=1)
    big = make_params(pa.HALF, pa.HALF, batch=520, **kw)
    one = make_params(pa.HALF, pa.HALF, batch=1, **kw)
    plan_big, plan_one = pa.Plan(big), pa.Plan(one)
    assert _plan_kernel(plan_big) == "depthwise direct", plan_big.describe()
    assert plan_big.buffer_bytes(capi.BUF_INPUT) > 2 ** 30
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(6)
    x = torch.randn((520, 112, 112, 96), generator=g, device=dev,
                    dtype=torch.float16)
    w = torch.randn((96, 1, 1, 3, 3), generator=g, device=dev,
                    dtype=torch.float16)

    def buf(plan, which):
        return torch.empty(max(plan.buffer_bytes(which), 16),
                           dtype=torch.uint8, device=dev)

    def run(plan, x_part):
        wp, out = buf(plan, capi.BUF_WEIGHTS_PACKED), buf(plan, capi.BUF_OUTPUT)
        plan.pack_weights(w.data_ptr(), wp.data_ptr())
        plan.fwd(x_part.data_ptr(), wp.data_ptr(), out.data_ptr())
        torch.cuda.synchronize()
        return out.view(torch.float16)

    got = run(plan_big, x).view(520, 56, 56, 96)
    for image in (0, 221, 222, 443, 444, 519):
        alone = run(plan_one, x[image].contiguous()).view(56, 56, 96)
        assert torch.equal(got[image], alone), image


PHASE_CASES = [
    # (input type, params, phases expected)
    # backward of 3x3 stride 2: phases of 1, 2, 2 and 4 taps
    (pa.HALF, dict(batch=2, field=(14, 15), kernel=(3, 3), ci=64, co=40,
                   idil=2, padLower=(1, 1), padUpper=(2, 2)), 4),
    # backward of 1x1 stride 2: one phase carries everything, three are zero
    (pa.HALF, dict(batch=2, field=(9, 10), kernel=(1, 1), ci=64, co=16,
                   idil=2, padUpper=(1, 1)), 4),
    # 7x7, dilated by 2 in both dimensions: 16 taps in the largest phase
    (pa.HALF, dict(batch=1, field=(12, 11), kernel=(7, 7), ci=8, co=24,
                   idil=2, pad=3), 4),
    # one dimension only; the other strides and has a dilated kernel
    (pa.HALF, dict(batch=2, field=(8, 13), kernel=(3, 3), ci=16, co=72,
                   idil=(3, 1), stride=(1, 2), kdil=(1, 2), pad=2, groups=2),
     3),
    # dilation 3 x 2, kernel dilation 2: phases without any tap in a dimension
    (pa.HALF, dict(batch=2, field=(7, 9), kernel=(3, 2), ci=16, co=136,
                   idil=(3, 2), pad=2, kdil=(2, 2)), 6),
    # truncation of the input under the dilation, negative effective padding
    (pa.HALF, dict(batch=2, field=(12, 12), kernel=(3, 3), ci=8, co=8, idil=2,
                   itl=(1, 2), itu=(2, 0), padLower=(0, 0),
                   padUpper=(0, 0)), 4),
    # few channels (padded copy), float and quarter operands
    (pa.HALF, dict(batch=4, field=(16, 16), kernel=(3, 3), ci=3, co=32,
                   idil=2, pad=1), 4),
    (pa.FLOAT, dict(batch=2, field=(9, 8), kernel=(3, 3), ci=8, co=16, idil=2,
                    pad=2), 4),
    (pa.QUARTER, dict(batch=2, field=(9, 8), kernel=(3, 3), ci=32, co=16,
                      idil=2, pad=2), 4),
    # three field dimensions: backward of a 3x3x3 stride-2 layer, and one
    # that strides in two of the three
    (pa.HALF, dict(batch=2, field=(4, 5, 6), kernel=(3, 3, 3), ci=16, co=24,
                   idil=2, padLower=(1, 1, 1), padUpper=(2, 2, 2)), 8),
    (pa.HALF, dict(batch=2, field=(5, 4, 6), kernel=(2, 3, 3), ci=8, co=40,
                   idil=(1, 2, 2), stride=(2, 1, 1), pad=1), 4),
]


@pytest.mark.parametrize("in_type,kw,phases", PHASE_CASES)
def test_igemm_phases_of_a_dilated_input(oracle, in_type, kw, phases):
    out_type = pa.FLOAT if in_type == pa.FLOAT else pa.HALF
    p = make_params(in_type, out_type, **kw)
    print("case", p, flush=True)
    if in_type == pa.QUARTER:
        got, want, plan = _fp8_case(oracle, p, 51, 1, 1)
    else:
        from gpu_helpers import quantize, run_conv
        acts, weights, biases = random_data(p, 51, "normal")
        aq, ad = quantize(acts, in_type)
        wq, wd = quantize(weights * 0.1, in_type)
        bq, bd = quantize(biases, out_type)
        got, plan = run_conv(p, aq, wq, bq, None, return_plan=True)
        want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert "%d phases" % phases in plan.describe(), plan.describe()
    assert rel_l2(got, want) <= (2e-6 if in_type == pa.FLOAT else 1e-3), \
        (rel_l2(got, want), plan.describe())


OUTPUT_PADDING_CASES = [
    dict(batch=2, field=(9, 8), kernel=(3, 3), ci=16, co=24, pad=1,
         opl=(1, 0), opu=(2, 3)),
    dict(batch=2, field=(12, 12), kernel=(3, 3), ci=8, co=40, stride=2,
         otl=(1, 0), opl=(0, 2), opu=(1, 0), groups=2),
    # what the backward pass of a strided 1x1 layer on an even field is: the
    # forward pass never read the last row and column
    dict(batch=2, field=(5, 5), kernel=(1, 1), ci=64, co=32, idil=2,
         opu=(1, 1)),
    dict(batch=2, field=(6, 7), kernel=(3, 3), ci=16, co=16, idil=2, pad=2,
         opl=(1, 1), opu=(0, 2)),
    # three field dimensions, padded in all of them; the backward pass of a
    # strided 1x1x1 layer on an even volume
    dict(batch=2, field=(4, 5, 6), kernel=(3, 3, 3), ci=8, co=16, pad=1,
         opl=(1, 0, 2), opu=(0, 1, 1)),
    dict(batch=2, field=(3, 3, 3), kernel=(1, 1, 1), ci=64, co=32, idil=2,
         opu=(1, 1, 1)),
]


@pytest.mark.parametrize("kw", OUTPUT_PADDING_CASES)
@pytest.mark.parametrize("bias", [False, True])
def test_igemm_output_padding(oracle, kw, bias):
    p = make_params(pa.HALF, pa.HALF, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 53, 1e-3, "implicit GEMM", wscale=0.1, bias=bias)


def test_igemm_phases_of_signs_are_exact(oracle):
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(9, 9), kernel=(3, 3),
                    ci=32, co=24, idil=2, pad=2)
    _run(oracle, p, 52, 0, "implicit GEMM", dist="pm1")


KERNEL_TRANSFORM_CASES = [
    # flipped in one dimension, in both; with a dilated kernel
    dict(batch=2, field=(9, 10), kernel=(3, 3), ci=16, co=24, pad=1,
         flipK=(True, False)),
    dict(batch=2, field=(9, 10), kernel=(3, 2), ci=64, co=72, pad=1,
         flipK=True, kdil=(1, 2)),
    # truncated (taps dropped at either end), truncated and flipped
    dict(batch=2, field=(12, 11), kernel=(5, 4), ci=8, co=40, pad=2,
         ktl=(1, 0), ktu=(1, 2)),
    dict(batch=2, field=(12, 11), kernel=(5, 4), ci=8, co=40, pad=2,
         ktl=(2, 1), ktu=(0, 1), flipK=(True, True), stride=2),
    # padded (the window is larger than the taps), padded and flipped
    dict(batch=2, field=(10, 10), kernel=(3, 3), ci=16, co=16, pad=2,
         kpl=(1, 0), kpu=(0, 2)),
    dict(batch=2, field=(10, 10), kernel=(3, 3), ci=16, co=16, pad=2,
         kpl=(1, 0), kpu=(0, 2), flipK=(True, True), kdil=2, groups=2),
    # together with a dilated input (phases) and with three dimensions
    dict(batch=2, field=(7, 8), kernel=(3, 3), ci=16, co=24, idil=2, pad=2,
         flipK=True, ktu=(1, 0)),
    dict(batch=2, field=(5, 6, 7), kernel=(3, 3, 3), ci=8, co=16, pad=1,
         flipK=(True, False, True), ktl=(0, 1, 0)),
]


@pytest.mark.parametrize("kw", KERNEL_TRANSFORM_CASES)
def test_igemm_kernel_truncation_padding_flip(oracle, kw):
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 71, 1e-3, "implicit GEMM", wscale=0.1)


STAGES_CASES = [
    # (params, input type, forced stages or None for the planner's choice)
    (dict(batch=3, field=(9, 11), kernel=(3, 3), ci=128, co=130, pad=1),
     pa.HALF, 2),
    (dict(batch=2, field=(7, 7), kernel=(3, 3), ci=40, co=72, pad=1),
     pa.HALF, 2),
    (dict(batch=2, field=(9, 11), kernel=(2, 3), ci=128, co=96, pad=1),
     pa.QUARTER, 2),
    # more workgroups than CUs: two stages are the planner's own choice
    (dict(batch=24, field=(40, 40), kernel=(1, 3), ci=16, co=128,
          padLower=(0, 1), padUpper=(0, 1)), pa.HALF, None),
]


@pytest.mark.parametrize("kw,in_type,stages", STAGES_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_igemm_two_stage_variant_matches_oracle(oracle, kw, in_type, stages,
                                                out_type):
    if in_type == pa.QUARTER and out_type == pa.FLOAT:
        pytest.skip("quarter inputs give half outputs")
    p = make_params(in_type, out_type, **kw)
    print("case", p, stages, flush=True)
    from gpu_helpers import quantize, run_conv
    options = None
    if stages:
        options = {"planConstraints": '{"gfx950": {"stages": %d}}' % stages}
    if in_type == pa.QUARTER:
        got, want, plan = _fp8_case(oracle, p, 12, 1, 0, options)
    else:
        acts, weights, biases = random_data(p, 12, "normal")
        aq, ad = quantize(acts, in_type)
        wq, wd = quantize(weights * 0.05, in_type)
        bq, bd = quantize(biases, out_type)
        got, plan = run_conv(p, aq, wq, bq, options, return_plan=True)
        want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert "LDS stages                 2" in plan.describe(), plan.describe()
    assert rel_l2(got, want) <= 1e-3, (rel_l2(got, want), plan.describe())


def test_igemm_split_k_of_signs_is_exact(oracle):
    # +-1 data: every partial sum is a small integer, so the parts add up
    # exactly whatever the cut
    p = make_params(pa.HALF, pa.FLOAT, batch=1, field=(5, 5), kernel=(3, 3),
                    ci=128, co=64, pad=1)
    _run(oracle, p, 9, 0, "implicit GEMM", dist="pm1", bias=False,
         options={"planConstraints": '{"gfx950": {"splitK": 5}}'})


def test_skinny_matmul_is_split_along_k():
    from test_matmul import run_matmul
    rng = np.random.default_rng(10)
    A = rng.standard_normal((1, 48, 4096)).astype(np.float16)
    B = (rng.standard_normal((1, 4096, 128)) / 64).astype(np.float16)
    got, plan = run_matmul(A, B, pa.HALF, pa.FLOAT, return_plan=True)
    assert "K split into parts" in plan.describe(), plan.describe()
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert rel_l2(got, want) <= 1e-5


DEPTHWISE_DILATED_CASES = [
    dict(batch=2, field=(7, 8), kernel=(3, 3), groups=16, idil=2,
         padLower=(1, 1), padUpper=(2, 2)),
    dict(batch=1, field=(5, 6), kernel=(4, 3), groups=40, idil=(3, 2), pad=2,
         kdil=(1, 2), stride=(2, 1)),
    dict(batch=3, field=(9,), kernel=(5,), groups=8, idil=4, itl=(1,),
         itu=(2,), pad=3),
]


@pytest.mark.parametrize("kw", DEPTHWISE_DILATED_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_depthwise_dilated_input_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, 7, "normal")
    aq, ad = quantize(acts, pa.HALF)
    wq, wd = quantize(weights, pa.HALF)
    bq, bd = quantize(biases, out_type)
    got, plan = run_conv(p, aq, wq, bq, return_plan=True)
    assert "dilated input" in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert rel_l2(got, want) <= 1e-3, (rel_l2(got, want), plan.describe())

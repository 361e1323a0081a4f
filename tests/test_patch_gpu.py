"""GPU parity of the matrix-core kernel that keeps a tile's input patch in LDS
(csrc/igemm_patch.hip) against the CPU oracle, through the C ABI.

Tolerances as for the other matrix-core tests: fp16 in / fp32 accumulate
relative L2 <= 1e-3 against the double-precision oracle fed the same rounded
inputs; fp8 <= 3e-2 (the only errors are accumulation and output rounding, so
1e-3 is asserted); +-1 data with fp32 output: exact.  The planner picks this
kernel by itself for unit-stride layers of at most one workgroup per CU; the
cases here force it where the planner would not."""
import json

import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, rel_l2

pytestmark = pytest.mark.gpu

FORCED = {"planConstraints": json.dumps({"gfx950": {"patch": 1}})}
FORCED64 = {"planConstraints":
            json.dumps({"gfx950": {"patch": 1, "blockM": 64}})}
FORCED16 = {"planConstraints": json.dumps({"gfx950": {"patch": 2}})}
PATCH = "input patch resident in LDS"
BLOCKS16 = "MFMA blocks of 16 pixels"


def _run(oracle, p, seed, tol, dist="normal", bias=True, options=FORCED,
         wscale=0.1, return_plan=False):
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, seed, dist)
    weights = weights * (1.0 if dist == "pm1" else wscale)
    aq, ad = quantize(acts, p.inputType)
    wq, wd = quantize(weights, p.inputType)
    bq, bd = quantize(biases, p.outputType)
    got, plan = run_conv(p, aq, wq, bq if bias else None, options,
                         return_plan=True)
    assert PATCH in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd if bias else None, threads=8)
    assert got.shape == want.shape
    if tol == 0:
        np.testing.assert_array_equal(got, want)
    else:
        err = rel_l2(got, want)
        assert err <= tol, (err, p)
    return (got, plan) if return_plan else got


CASES = [
    # the ResNet-style 3x3 layer at a small batch; a tile crosses images
    dict(batch=3, field=(28, 28), kernel=(3, 3), ci=128, co=128, pad=1),
    # one slice of channels, output channels ragged against 128, M ragged
    dict(batch=2, field=(13, 11), kernel=(3, 3), ci=64, co=72, pad=1),
    # three slices, groups, a 1 x 3 kernel with asymmetric padding
    dict(batch=2, field=(9, 14), kernel=(1, 3), ci=192, co=40, groups=2,
         padLower=(0, 2), padUpper=(0, 0)),
    # tiny images: a tile spans many of them, padding rows in between
    dict(batch=40, field=(5, 4), kernel=(3, 3), ci=64, co=136, pad=1),
    # kernel dilation and more padding than the window needs
    dict(batch=2, field=(12, 12), kernel=(3, 3), ci=64, co=128, kdil=(2, 1),
         pad=2),
    # a wide kernel: 49 taps x 2 slices = 98 k-steps (more than one table of
    # tap offsets)
    dict(batch=1, field=(16, 16), kernel=(7, 7), ci=128, co=128, pad=3),
    # input truncation (negative padding) and a kernel flipped and truncated
    dict(batch=2, field=(14, 14), kernel=(4, 3), ci=64, co=128, itl=(1, 0),
         itu=(0, 2), ktl=(1, 0), flipK=(True, True), pad=1),
    # pointwise, forced onto this kernel: one tap
    dict(batch=2, field=(10, 10), kernel=(1, 1), ci=128, co=128),
    # a 1-D field
    dict(batch=4, field=(50,), kernel=(5,), ci=64, co=96, pad=2),
]


@pytest.mark.parametrize("kw", CASES)
def test_patch_fp16_matches_oracle(oracle, kw):
    p = make_params(pa.HALF, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 11, 1e-3)


@pytest.mark.parametrize("kw", CASES[1:5])
def test_patch_fp16_in_fp32_out_pm1_exact(oracle, kw):
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 12, 0, dist="pm1")


@pytest.mark.parametrize("kw", CASES[:4])
def test_patch_64_row_tiles(oracle, kw):
    p = make_params(pa.HALF, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 13, 1e-3, options=FORCED64, bias=False)


def _forced16(tile_pixels):
    return {"planConstraints": json.dumps(
        {"gfx950": {"patch": 2, "blockM": tile_pixels}})}


# (the pointwise case has one tap: the wave pairs of this variant take turns
# by k-step, which wants two)
@pytest.mark.parametrize("kw", [c for c in CASES if c["kernel"] != (1, 1)])
def test_patch_16_pixel_blocks(oracle, kw):
    p = make_params(pa.HALF, **kw)
    print("case", p, flush=True)
    _, plan = _run(oracle, p, 14, 1e-3, options=FORCED16, return_plan=True)
    assert BLOCKS16 in plan.describe()


@pytest.mark.parametrize("tile_pixels", [112, 98, 37, 16, 5])
def test_patch_16_pixel_blocks_tile_heights(oracle, tile_pixels):
    p = make_params(pa.HALF, pa.FLOAT, **CASES[1])
    print("case", p, tile_pixels, flush=True)
    _, plan = _run(oracle, p, 15, 0, dist="pm1",
                   options=_forced16(tile_pixels), return_plan=True)
    assert BLOCKS16 in plan.describe()
    assert "block M x N x K            %d x" % tile_pixels in plan.describe()


@pytest.mark.parametrize("kw", CASES[2:7])
def test_patch_16_pixel_blocks_pm1_exact(oracle, kw):
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 16, 0, dist="pm1", options=FORCED16)


# Who loads which part of the patch: slice 0 goes to all eight waves before
# the first barrier, the later slices to the older wave of each SIMD behind
# it.  The cases: more column blocks per row than waves (a 56-wide field: ten
# of them), a single block per row with eight slices, and a row of three
# blocks with four slices - each with a tile height that makes the rows of
# the patch ragged against the tiles.
@pytest.mark.parametrize("kw,tile_pixels", [
    (dict(batch=2, field=(12, 56), kernel=(3, 3), ci=128, co=128, pad=1), 0),
    (dict(batch=2, field=(12, 56), kernel=(3, 3), ci=128, co=128, pad=1), 112),
    (dict(batch=6, field=(4, 4), kernel=(3, 3), ci=256, co=64, pad=1), 48),
    (dict(batch=3, field=(9, 17), kernel=(3, 3), ci=256, co=136, pad=1), 0),
    (dict(batch=3, field=(9, 17), kernel=(3, 3), ci=256, co=136, pad=1), 80),
])
def test_patch_later_slices_loaded_by_the_older_waves(oracle, kw, tile_pixels):
    """tile_pixels 0: the 32-pixel-block kernel, else the 16-pixel-block one
    with tiles of that many pixels."""
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, tile_pixels, flush=True)
    opts = _forced16(tile_pixels) if tile_pixels else FORCED
    _, plan = _run(oracle, p, 18, 0, dist="pm1", options=opts,
                   return_plan=True)
    assert PATCH in plan.describe()
    assert (BLOCKS16 in plan.describe()) == bool(tile_pixels)


def test_patch_16_pixel_blocks_refuse_one_tap():
    p = make_params(pa.HALF, **CASES[7])
    assert PATCH not in pa.Plan(p, FORCED16).describe()


@pytest.mark.parametrize("options", [FORCED, FORCED16])
def test_patch_that_leaves_no_room_beside_it(oracle, options):
    """Four channel slices of a 28-wide field: the patch takes 140 KB of the
    160, so the waves' sums meet in its place once everybody has left it."""
    p = make_params(pa.HALF, batch=2, field=(28, 28), kernel=(3, 3), ci=256,
                    co=136, pad=1)
    print("case", p, flush=True)
    _run(oracle, p, 17, 1e-3, options=options)


def test_patch_is_the_planners_choice_for_the_benchmark_layers():
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    assert PATCH in pa.Plan(p).describe()
    p = make_params(pa.QUARTER, pa.HALF, batch=64, field=(14, 14),
                    kernel=(3, 3), ci=256, co=256, pad=1)
    assert PATCH in pa.Plan(p).describe()
    # more workgroups than CUs: tiles of 112 pixels, several rounds of them
    p = make_params(pa.HALF, batch=256, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    text = pa.Plan(p).describe()
    assert BLOCKS16 in text and "block M x N x K            112 x" in text
    # channels that do not come in whole 128-byte slices: the streaming kernel
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=96,
                    co=128, pad=1)
    assert PATCH not in pa.Plan(p).describe()
    off = {"planConstraints": json.dumps({"gfx950": {"patch": 0}})}
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    assert PATCH not in pa.Plan(p, off).describe()


def test_patch_forced_on_a_strided_layer_is_refused_quietly():
    # the constraint asks "whenever it can": a strided layer stays where it was
    p = make_params(pa.HALF, batch=2, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1, stride=2)
    assert PATCH not in pa.Plan(p, FORCED).describe()


@pytest.mark.parametrize("options", [FORCED, FORCED16])
@pytest.mark.parametrize("fmt_a,fmt_w", [(1, 1), (1, 0), (0, 1), (0, 0)])
def test_patch_fp8_matches_oracle(oracle, fmt_a, fmt_w, options):
    from test_fast_gpu import _fp8_case
    p = make_params(pa.QUARTER, pa.HALF, batch=5, field=(14, 14),
                    kernel=(3, 3), ci=256, co=256, pad=1)
    got, want, plan = _fp8_case(oracle, p, 6, fmt_a, fmt_w, options=options)
    assert PATCH in plan.describe()
    err = rel_l2(got, want)
    assert err <= 3e-2, err
    assert err <= 1e-3, err


@pytest.mark.parametrize("options", [FORCED, FORCED16])
def test_patch_fp8_ragged(oracle, options):
    from test_fast_gpu import _fp8_case
    p = make_params(pa.QUARTER, pa.HALF, batch=3, field=(7, 9), kernel=(3, 2),
                    ci=128, co=40, groups=2, pad=1)
    got, want, plan = _fp8_case(oracle, p, 7, 1, 1, options=options)
    assert PATCH in plan.describe()
    assert rel_l2(got, want) <= 1e-3


def test_patch_twice_in_a_row_is_bit_identical(oracle):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.HALF, **CASES[0])
    acts, weights, _ = random_data(p, 21, "normal")
    aq, _ = quantize(acts, p.inputType)
    wq, _ = quantize(weights * 0.1, p.inputType)
    first = run_conv(p, aq, wq, None, FORCED)
    second = run_conv(p, aq, wq, None, FORCED)
    np.testing.assert_array_equal(first, second)


def test_patch_small_patch_float_output_repeats(oracle):
    """A patch smaller than the fp32 output tile: the epilogue's exchange area
    and the output tile must not share LDS (waves leave the exchange at
    different times).  Many runs, all equal to the oracle's +-1 result."""
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(6, 7), kernel=(3, 3),
                    ci=64, co=72, pad=1)
    first = _run(oracle, p, 41, 0, dist="pm1")
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, 41, "pm1")
    aq, _ = quantize(acts, p.inputType)
    wq, _ = quantize(weights, p.inputType)
    bq, _ = quantize(biases, p.outputType)
    for _ in range(20):
        np.testing.assert_array_equal(run_conv(p, aq, wq, bq, FORCED), first)

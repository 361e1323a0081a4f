"""Inputs of 1 to 4 channels (images, waveforms) on the matrix cores without
padding the channels: a kernel row's kW * Ci neighbouring elements fill
k-steps in chunks of 8 (role of the reference's planner choosing a small inChansPerGroup for
the first layer, lib/poplin/ConvPlan.cpp:1065-1238, and of the input
rearrangement it costs there).  Parity against the oracle through the C ABI."""
import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, rel_l2

pytestmark = pytest.mark.gpu

THIN = "kernel rows as k-steps"
# (by name: the planner leaves layers of little work to the generic kernel)
FORCED = {"planConstraints": '{"gfx950": {"thinInput": 1}}'}

CASES = [
    # the 7 x 7 stride-2 first layer of a ResNet, small
    dict(batch=2, field=(64, 64), kernel=(7, 7), ci=3, co=64, pad=3, stride=2),
    # unit stride over three channels: windows start at odd element offsets
    dict(batch=3, field=(20, 22), kernel=(3, 3), ci=3, co=32, pad=1),
    dict(batch=2, field=(17, 16), kernel=(5, 5), ci=4, co=48, pad=2),
    # one channel, a kernel wider than high, strides that differ
    dict(batch=2, field=(12, 40), kernel=(3, 9), ci=1, co=16,
         padLower=(1, 4), padUpper=(1, 4), stride=(1, 2)),
    # asymmetric padding, a stride that skips pixels
    dict(batch=2, field=(30, 31), kernel=(7, 7), ci=2, co=64,
         padLower=(2, 1), padUpper=(0, 3), stride=3),
    # one dimension (a waveform)
    dict(batch=4, field=(200,), kernel=(9,), ci=2, co=16, pad=4, stride=2),
    dict(batch=2, field=(334,), kernel=(31,), ci=1, co=32, pad=15, stride=5),
    # rows that are no whole 16-byte vector (copied in dwords)
    dict(batch=2, field=(9, 11), kernel=(3, 3), ci=2, co=16, pad=1),
    # two and four kernel rows (run as three and five), six (as seven)
    dict(batch=2, field=(10, 12), kernel=(2, 5), ci=3, co=16, padLower=(0, 2),
         padUpper=(1, 2)),
    dict(batch=1, field=(12, 12), kernel=(4, 4), ci=4, co=32, pad=1,
         stride=2),
    dict(batch=1, field=(14, 16), kernel=(6, 3), ci=3, co=64, pad=1),
    # more than seven kernel rows of few elements: chunks of several rows
    # share a k-step
    dict(batch=2, field=(20, 18), kernel=(9, 4), ci=1, co=16, pad=2),
    dict(batch=1, field=(30, 30), kernel=(11, 11), ci=1, co=32, pad=5,
         stride=2),
    dict(batch=2, field=(16, 16), kernel=(14, 2), ci=4, co=16,
         padLower=(6, 0), padUpper=(7, 1)),
    # more tiles than workgroups: the persistent loop goes round
    dict(batch=40, field=(64, 32), kernel=(3, 3), ci=3, co=16, pad=1),
    # no padding at all; an output narrower than a block of 16 pixels
    dict(batch=2, field=(9, 8), kernel=(3, 3), ci=4, co=16),
    # as much padding as the kernel reaches
    dict(batch=1, field=(8, 8), kernel=(3, 3), ci=2, co=16, pad=2),
    # input truncation: rows and columns that read as zeros
    dict(batch=2, field=(12, 14), kernel=(3, 3), ci=3, co=16, itl=(1, 2),
         itu=(2, 1), pad=2),
]


@pytest.mark.parametrize("kw", CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_thin_input_matches_oracle(oracle, kw, out_type):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    acts, weights, biases = random_data(p, 41, "normal")
    aq, ad = quantize(acts, pa.HALF)
    wq, wd = quantize(weights * 0.2, pa.HALF)
    bq, bd = quantize(biases, out_type)
    got, plan = run_conv(p, aq, wq, bq, FORCED, return_plan=True)
    assert THIN in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    tol = 1e-3 if out_type == pa.HALF else 1e-5
    assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())


@pytest.mark.parametrize("kw", [CASES[0], CASES[1], CASES[6], CASES[11]])
def test_thin_input_of_signs_is_exact(oracle, kw):
    # +-1 tensors: every product and every sum is a small integer
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    acts, weights, _ = random_data(p, 42, "normal")
    aq, ad = quantize(np.sign(acts) + (acts == 0), pa.HALF)
    wq, wd = quantize(np.sign(weights) + (weights == 0), pa.HALF)
    got, plan = run_conv(p, aq, wq, None, FORCED, return_plan=True)
    assert THIN in plan.describe(), plan.describe()
    np.testing.assert_array_equal(got, oracle.convolution(p, ad, wd,
                                                          threads=8))


def test_thin_input_does_not_spread_an_infinity(oracle):
    # The operand of a block's last lanes reaches past the kernel row into the
    # next pixels; those elements are masked, not multiplied by zero weights:
    # an infinity next to a window stays out of its sum.
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.HALF, pa.FLOAT, batch=1, field=(8, 40), kernel=(3, 3),
                    ci=3, co=16, pad=1)
    acts, weights, _ = random_data(p, 43, "normal")
    acts[0, 1, 4, 20] = np.inf
    aq, ad = quantize(acts, pa.HALF)
    wq, wd = quantize(weights, pa.HALF)
    got, plan = run_conv(p, aq, wq, None, FORCED, return_plan=True)
    assert THIN in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, threads=8)
    finite = np.isfinite(want)
    # the windows that cover the element: 3 x 3 of them, every channel
    assert (~finite).sum() == 9 * 16
    np.testing.assert_array_equal(np.isfinite(got), finite)
    assert rel_l2(got[finite], want[finite]) <= 1e-5


def test_thin_input_is_the_planners_choice_for_a_first_layer():
    stem = make_params(pa.HALF, batch=32, field=(224, 224), kernel=(7, 7),
                       ci=3, co=64, pad=3, stride=2)
    text = pa.Plan(stem).describe()
    assert THIN in text and "workspaceBytes             0" in text
    # named kernels and tiles keep the padded copy
    named = {"planConstraints": '{"gfx950": {"kernel": "igemm"}}'}
    assert "input channels padded      3 -> 8" in pa.Plan(stem,
                                                          named).describe()


def _random_thin_case(r):
    """A random layer within what the kernel takes (or close to it: what the
    canonical form then moves outside - padded outputs, say - is skipped)."""
    ci = r.choice([1, 2, 3, 3, 4])
    kw = r.randint(1, 32 // ci)
    kh = r.randint(1, min(10, 28 // ((kw * ci + 7) // 8)))
    if kh * kw < 2:
        kh = 2
    one_d = r.random() < 0.15
    if one_d:
        kh = None
    width = r.randint(kw, kw + 40)
    if (width * ci) % 2:
        width += 1
    field = (width,) if one_d else (r.randint(kh, kh + 24), width)
    kernel = (kw,) if one_d else (kh, kw)
    n = len(field)
    kw_args = dict(
        batch=r.randint(1, 5), field=field, kernel=kernel, ci=ci,
        co=r.choice([16, 32, 48, 64]),
        stride=[r.choice([1, 1, 2, 2, 3, 4]) for _ in range(n)],
        # (no window wholly in the border: that is output padding)
        padLower=[r.randint(0, min(4, k - 1)) for k in kernel],
        padUpper=[r.randint(0, min(4, k - 1)) for k in kernel])
    if r.random() < 0.2:
        kw_args["itl"] = [r.randint(0, 1) for _ in range(n)]
        kw_args["itu"] = [r.randint(0, 1) for _ in range(n)]
    return kw_args


def test_thin_input_random_params(oracle):
    import random
    from gpu_helpers import quantize, run_conv
    from poplibs_amd.capi import MxconvError
    r = random.Random(44)
    ran = 0
    for case in range(260):
        kw = _random_thin_case(r)
        out_type = r.choice([pa.HALF, pa.FLOAT])
        try:
            p = make_params(pa.HALF, out_type, **kw)
            p.validate()
            plan = pa.Plan(p, FORCED)
        except MxconvError:
            continue  # (not a layer, or not this kernel's after canonicalize)
        print("case", case, kw, flush=True)
        acts, weights, biases = random_data(p, 100 + case, "normal")
        aq, ad = quantize(acts, pa.HALF)
        wq, wd = quantize(weights * 0.2, pa.HALF)
        bq, bd = quantize(biases, out_type)
        got = run_conv(p, aq, wq, bq, plan=plan)
        assert THIN in plan.describe()
        want = oracle.convolution(p, ad, wd, bd, threads=8)
        tol = 1e-3 if out_type == pa.HALF else 1e-5
        assert rel_l2(got, want) <= tol, (case, kw, rel_l2(got, want))
        ran += 1
    assert ran >= 150, ran

"""GPU parity of the any-parameter direct kernel against the CPU oracle, all
through the C ABI.  Tolerances: fp32 in / fp32 accumulate rel-L2 <= 1e-5;
fp16 in / fp32 accumulate / fp16 out rel-L2 <= 1e-3; +-1 data exact."""
import random

import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, random_params, rel_l2

pytestmark = pytest.mark.gpu

GENERIC = {"planConstraints": '{"gfx950": {"kernel": "generic"}}'}


def _check(oracle, p, seed, tol, dist="uniform", bias=True, options=GENERIC):
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, seed, dist)
    aq, ad = quantize(acts, p.inputType)
    wq, wd = quantize(weights, p.inputType)
    bq, bd = quantize(biases, p.outputType)
    want = oracle.convolution(p, ad, wd, bd if bias else None)
    got = run_conv(p, aq, wq, bq if bias else None, options)
    assert got.shape == want.shape
    if tol == 0:
        np.testing.assert_array_equal(got, want)
    else:
        err = rel_l2(got, want)
        assert err <= tol, (err, p)
    return got, want


@pytest.mark.parametrize("seed", range(40))
def test_generic_fuzz_fp32(oracle, seed):
    p = random_params(random.Random(1000 + seed), pa.FLOAT)
    print("case", seed, p, flush=True)
    _check(oracle, p, seed, 1e-5)


@pytest.mark.parametrize("seed", range(20))
def test_generic_fuzz_fp16(oracle, seed):
    p = random_params(random.Random(2000 + seed), pa.HALF)
    print("case", seed, p, flush=True)
    _check(oracle, p, seed, 1e-3)


@pytest.mark.parametrize("seed", range(10))
def test_generic_fuzz_fp16_in_fp32_out_pm1_exact(oracle, seed):
    """The harness's zero-tolerance mode: +-1 data, exactly representable
    sums (tools/single_conv_layer.cpp:979-1005)."""
    p = random_params(random.Random(3000 + seed), pa.HALF, pa.FLOAT)
    print("case", seed, p, flush=True)
    _check(oracle, p, seed, 0, dist="pm1")


def test_generic_baseline_config1(oracle):
    """N=1 32x32 Cin=Cout=16 3x3 s1 p1 fp32, uniform[-1,1) seed 0."""
    p = make_params(pa.FLOAT, field=(32, 32), kernel=(3, 3), ci=16, co=16,
                    pad=1)
    assert p.getFwdFlops() == 4524032
    _check(oracle, p, 0, 1e-5, bias=False)


@pytest.mark.parametrize("kw", [
    dict(batch=0, field=(4, 4), kernel=(3, 3), ci=2, co=2, pad=1),
    dict(field=(4, 4), kernel=(3, 3), ci=0, co=2, pad=1),
    dict(field=(4, 4), kernel=(3, 3), ci=2, co=0, pad=1),
    dict(field=(), kernel=(), ci=3, co=2, batch=2),           # 0-D field
    dict(field=(9,), kernel=(3,), ci=2, co=2, stride=2),      # 1-D
    dict(field=(3, 4, 5), kernel=(2, 2, 2), ci=2, co=2, pad=1),  # 3-D
    dict(field=(2, 3, 2, 3), kernel=(1, 2, 1, 2), ci=1, co=2),  # 4-D
    # all-zero output (kernel entirely in the padding)
    dict(field=(2,), kernel=(1,), padLower=4, otu=4),
    # negative padding via truncation, output padding, flips
    dict(field=(8, 8), kernel=(3, 3), itl=(1, 2), itu=(2, 0), opl=(1, 0),
         opu=(0, 2), flipIn=(True, False), flipK=(False, True), ci=2, co=2),
    # input dilation sharing a factor with the stride
    dict(field=(6, 6), kernel=(3, 3), idil=(2, 4), stride=(2, 2), pad=2, ci=2,
         co=3),
])
def test_generic_edge_cases(oracle, kw):
    p = make_params(pa.FLOAT, **kw)
    _check(oracle, p, 5, 1e-5)


def test_generic_run_to_run_bit_identical(oracle):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.HALF, field=(14, 14), kernel=(3, 3), ci=8, co=8, pad=1,
                    batch=2)
    acts, weights, _ = random_data(p, 11, "normal")
    aq, _ = quantize(acts, p.inputType)
    wq, _ = quantize(weights, p.inputType)
    a = run_conv(p, aq, wq, None, GENERIC)
    b = run_conv(p, aq, wq, None, GENERIC)
    assert np.array_equal(a, b)

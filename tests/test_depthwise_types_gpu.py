"""Depthwise layers of fp32 and fp8 inputs (the LDS-tiled kernel with 16-byte
vectors of 4 or 16 channels) against the CPU oracle, through the C ABI.
fp32 in and out, +-1 data: exact; otherwise relative L2 <= 1e-3 (fp32 in,
half out; fp8 in, half out - every fp8 product is exact in fp32)."""
import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, rel_l2

pytestmark = pytest.mark.gpu
KERNEL = "depthwise direct"

CASES = [
    dict(batch=2, field=(28, 29), kernel=(3, 3), groups=32, pad=1),
    dict(batch=2, field=(17, 15), kernel=(3, 3), groups=48, pad=1, stride=2),
    dict(batch=1, field=(13, 13), kernel=(5, 5), groups=16, pad=2),
    dict(batch=3, field=(9, 20), kernel=(3, 2), groups=80, padLower=(1, 0),
         padUpper=(0, 1), kdil=(2, 1)),
    dict(batch=2, field=(7, 7), kernel=(7, 7), groups=64, pad=3),
    dict(batch=2, field=(30,), kernel=(5,), groups=16, pad=2, stride=2),
]


@pytest.mark.parametrize("kw", CASES)
@pytest.mark.parametrize("out_type", [pa.FLOAT, pa.HALF])
def test_depthwise_fp32_matches_oracle(oracle, kw, out_type):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.FLOAT, out_type, **kw)
    print("case", p, flush=True)
    exact = out_type == pa.FLOAT
    acts, weights, biases = random_data(p, 61, "pm1" if exact else "normal")
    aq, ad = quantize(acts, pa.FLOAT)
    wq, wd = quantize(weights, pa.FLOAT)
    bq, bd = quantize(biases, out_type)
    got, plan = run_conv(p, aq, wq, bq, None, return_plan=True)
    assert KERNEL in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    if exact:
        np.testing.assert_array_equal(got, want)
    else:
        assert rel_l2(got, want) <= 1e-3


def test_depthwise_fp32_channels_in_vectors_of_four(oracle):
    """12 channels: three vectors of fp32, no whole vector of eight."""
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.FLOAT, pa.FLOAT, batch=2, field=(9, 9), kernel=(3, 3),
                    groups=12, pad=1)
    acts, weights, _ = random_data(p, 62, "pm1")
    got, plan = run_conv(p, quantize(acts, pa.FLOAT)[0],
                         quantize(weights, pa.FLOAT)[0], None, None,
                         return_plan=True)
    assert KERNEL in plan.describe()
    np.testing.assert_array_equal(
        got, oracle.convolution(p, acts, weights, threads=8))
    # 10 channels: the generic kernel
    p = make_params(pa.FLOAT, pa.FLOAT, batch=2, field=(9, 9), kernel=(3, 3),
                    groups=10, pad=1)
    assert KERNEL not in pa.Plan(p).describe()


@pytest.mark.parametrize("kw", CASES)
@pytest.mark.parametrize("fmt_a,fmt_w", [(1, 1), (1, 0), (0, 1), (0, 0)])
def test_depthwise_fp8_matches_oracle(oracle, kw, fmt_a, fmt_w):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.QUARTER, pa.HALF, **kw)
    print("case", p, fmt_a, fmt_w, flush=True)
    acts, weights, biases = random_data(p, 63, "normal")
    weights = weights * 0.2

    def scale_for(x, fmt):
        maxv = 448.0 if fmt == oracle.E4M3 else 57344.0
        return int(np.ceil(np.log2(np.abs(x).max() / maxv)))

    sa, sw = scale_for(acts, fmt_a), scale_for(weights, fmt_w)
    aq, ad = quantize(acts, pa.QUARTER, oracle, fmt_a, sa)
    wq, wd = quantize(weights, pa.QUARTER, oracle, fmt_w, sw)
    bq, bd = quantize(biases, pa.HALF)
    got, plan = run_conv(p, aq, wq, bq, None,
                         in_meta=pa.quarter_metadata(fmt_a, sa),
                         w_meta=pa.quarter_metadata(fmt_w, sw),
                         return_plan=True)
    assert KERNEL in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    assert rel_l2(got, want) <= 1e-3


def test_depthwise_quarter_fixtures_plan_the_depthwise_kernel():
    """The reference's own quarter depthwise layers
    (tests/poplin/json/depthwise_conv_quarter{1,2}.json)."""
    import os
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    for name in ("depthwise_conv_quarter1.json", "depthwise_conv_quarter2.json"):
        p = pa.ConvParams.from_json(open(os.path.join(golden, name)).read())
        text = pa.Plan(p).describe()
        print(name, [l for l in text.splitlines() if "kernel  " in l])


@pytest.mark.parametrize("kw", [
    # the backward pass of strided depthwise layers: the deltas dilated by the
    # stride (3 x 3 and 5 x 5 at stride 2, a stride of 3, uneven strides)
    dict(batch=2, field=(14, 15), kernel=(3, 3), groups=32, idil=2, pad=1),
    dict(batch=2, field=(9, 8), kernel=(5, 5), groups=16, idil=2, pad=3),
    dict(batch=1, field=(7, 9), kernel=(3, 3), groups=20, idil=(3, 1), pad=2),
])
@pytest.mark.parametrize("out_type", [pa.FLOAT, pa.HALF])
def test_depthwise_fp32_dilated_input(oracle, kw, out_type):
    from gpu_helpers import quantize, run_conv
    p = make_params(pa.FLOAT, out_type, **kw)
    print("case", p, flush=True)
    exact = out_type == pa.FLOAT
    acts, weights, biases = random_data(p, 64, "pm1" if exact else "normal")
    got, plan = run_conv(p, quantize(acts, pa.FLOAT)[0],
                         quantize(weights, pa.FLOAT)[0],
                         quantize(biases, out_type)[0], None,
                         return_plan=True)
    assert KERNEL in plan.describe(), plan.describe()
    want = oracle.convolution(p, acts, weights,
                              quantize(biases, out_type)[1], threads=8)
    if exact:
        np.testing.assert_array_equal(got, want)
    else:
        assert rel_l2(got, want) <= 1e-3

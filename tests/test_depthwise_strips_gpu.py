"""Depthwise layers with a 7 x 7 kernel (unit stride and dilation): the
LDS-tiled kernel's strips of neighbouring output pixels per thread, against
the CPU oracle.  +-1 data, fp32 output: exact; half output <= 1e-3."""
import json

import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, rel_l2

pytestmark = pytest.mark.gpu


def _run(oracle, p, seed, tol, options=None, bias=True):
    from gpu_helpers import quantize, run_conv
    dist = "pm1" if tol == 0 else "normal"
    acts, weights, biases = random_data(p, seed, dist)
    if tol != 0:
        weights = weights * 0.1
    aq, ad = quantize(acts, p.inputType)
    wq, wd = quantize(weights, p.inputType)
    bq, bd = quantize(biases, p.outputType)
    got, plan = run_conv(p, aq, wq, bq if bias else None, options,
                         return_plan=True)
    assert "depthwise direct" in plan.describe(), plan.describe()
    want = oracle.convolution(p, ad, wd, bd if bias else None, threads=8)
    if tol == 0:
        np.testing.assert_array_equal(got, want)
    else:
        assert rel_l2(got, want) <= tol
    return plan


CASES = [
    # ConvNeXt's stages at a small batch: tiles of 14 and 7 columns (strips
    # of seven pixels), 12 / 24 / 48 channel vectors (one block, a block and
    # a half, three)
    dict(batch=2, field=(56, 56), kernel=(7, 7), groups=96, pad=3),
    dict(batch=2, field=(28, 28), kernel=(7, 7), groups=192, pad=3),
    dict(batch=3, field=(14, 14), kernel=(7, 7), groups=384, pad=3),
    dict(batch=3, field=(7, 7), kernel=(7, 7), groups=768, pad=3),
    # widths that are no multiple of seven (strips of four, the last one of a
    # tile and of the field partial), heights ragged against the tile
    dict(batch=2, field=(19, 13), kernel=(7, 7), groups=40, pad=3),
    dict(batch=1, field=(11, 30), kernel=(7, 7), groups=8, pad=3),
    # unpadded and unevenly padded
    dict(batch=2, field=(20, 17), kernel=(7, 7), groups=16),
    dict(batch=2, field=(9, 12), kernel=(7, 7), groups=24, padLower=(5, 0),
         padUpper=(1, 6)),
]


@pytest.mark.parametrize("kw", CASES)
@pytest.mark.parametrize("out_type", [pa.FLOAT, pa.HALF])
def test_depthwise_7x7_matches_oracle(oracle, kw, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 51, 0 if out_type == pa.FLOAT else 1e-3,
         bias=kw["groups"] % 16 == 0)


@pytest.mark.parametrize("tile", [(3, 7), (5, 14), (2, 9), (4, 4), (1, 1)])
def test_depthwise_7x7_forced_tiles(oracle, tile):
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(16, 15), kernel=(7, 7),
                    groups=32, pad=3)
    options = {"planConstraints": json.dumps(
        {"gfx950": {"tileH": tile[0], "tileW": tile[1]}})}
    _run(oracle, p, 52, 0, options=options)

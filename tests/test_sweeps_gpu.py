"""Seeded sweeps of random layers through the kernels a planner picks for
speed, on data of +-1 (and 0 where padding supplies it): every product and
every partial sum is a small integer, so the fp32 results must equal the
double-precision oracle's exactly, whatever order a kernel sums in.  The
reference draws its random convolutions the same way
(tools/single_conv_layer_random.py:213-370 for the parameter ranges,
lib/poplibs_test/Util.cpp:42-60 for the +-1 data); the harness-level sweep of
those is test_harness.py's, this one aims at the shapes the matrix-core,
pointwise and depthwise kernels take, which that generator's FLOP cap rarely
reaches."""
import collections
import json
import random

import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data

pytestmark = pytest.mark.gpu


def _exact(oracle, p, options, seed):
    from gpu_helpers import quantize, run_conv
    acts, weights, biases = random_data(p, seed, "pm1")
    aq, ad = quantize(acts, p.inputType, oracle)
    wq, wd = quantize(weights, p.inputType, oracle)
    bq, bd = quantize(biases, p.outputType, oracle)
    got = run_conv(p, aq, wq, bq, options)
    want = oracle.convolution(p, ad, wd, bd, threads=8)
    np.testing.assert_array_equal(got, want)


def _pads(rng, field, most):
    return (tuple(rng.randint(0, most) for _ in field),
            tuple(rng.randint(0, most) for _ in field))


def test_resident_patch_kernels_random_layers(oracle):
    """Both variants forced through planConstraints, tile heights of the
    16-pixel variant drawn too."""
    rng = random.Random(20250611)
    ran = collections.Counter()
    for case in range(400):
        field = tuple(rng.randint(1, 20)
                      for _ in range(rng.choice([1, 2, 2, 2])))
        kernel = tuple(rng.randint(1, min(5, f + 2)) for f in field)
        lo, hi = _pads(rng, field, 3)
        kw = dict(batch=rng.randint(1, 12), field=field, kernel=kernel,
                  ci=rng.choice([64, 128, 192, 256]),
                  co=rng.choice([8, 16, 40, 64, 128, 136, 200, 264]),
                  groups=rng.choice([1, 1, 1, 2, 3]), padLower=lo,
                  padUpper=hi)
        if rng.random() < 0.3:
            kw["kdil"] = tuple(rng.randint(1, 3) for _ in field)
        if rng.random() < 0.2:
            kw["flipK"] = tuple(rng.random() < 0.5 for _ in field)
        if rng.random() < 0.15:
            kw["itl"] = tuple(rng.randint(0, 1) for _ in field)
        if rng.random() < 0.15:
            kw["ktu"] = tuple(rng.randint(0, 1) for _ in field)
        variant = rng.choice([1, 2, 2])
        constraints = {"patch": variant}
        if variant == 2 and rng.random() < 0.6:
            constraints["blockM"] = rng.randint(1, 112)
        if variant == 1 and rng.random() < 0.5:
            constraints["blockM"] = 64
        options = {"planConstraints": json.dumps({"gfx950": constraints})}
        try:
            p = make_params(pa.HALF, pa.FLOAT, **kw)
            plan = pa.Plan(p, options)
        except pa.MxconvError:
            continue  # a layer the variant refuses, or no valid convolution
        if "input patch resident in LDS" not in plan.describe():
            continue
        print("case", case, kw, constraints, flush=True)
        _exact(oracle, p, options, 1000 + case)
        ran[variant] += 1
    assert ran[1] >= 30 and ran[2] >= 60, ran


def test_planners_choice_random_layers(oracle):
    """Pointwise, depthwise and dense layers as the planner runs them."""
    rng = random.Random(20250612)
    kernels = collections.Counter()
    for case in range(300):
        kind = rng.choice(["pointwise", "depthwise", "dense", "dense"])
        if kind == "pointwise":
            kw = dict(batch=rng.randint(1, 6),
                      field=(rng.randint(1, 30), rng.randint(1, 30)),
                      kernel=(1, 1), ci=16 * rng.randint(1, 16),
                      co=8 * rng.randint(1, 40), groups=rng.choice([1, 1, 2]))
            if rng.random() < 0.3:
                kw["stride"] = (rng.randint(1, 2), rng.randint(1, 2))
        elif kind == "depthwise":
            k = rng.choice([(3, 3), (3, 3), (5, 5), (3, 1), (2, 2)])
            lo, hi = _pads(rng, k, 2)
            s = rng.choice([1, 1, 2])
            kw = dict(batch=rng.randint(1, 4),
                      field=(rng.randint(3, 40), rng.randint(3, 40)),
                      kernel=k, ci=1, co=1, groups=8 * rng.randint(1, 28),
                      padLower=lo, padUpper=hi, stride=(s, s))
            if rng.random() < 0.2:
                kw["kdil"] = (rng.randint(1, 2), rng.randint(1, 2))
        else:
            k = (rng.randint(1, 4), rng.randint(1, 4))
            lo, hi = _pads(rng, k, 2)
            kw = dict(batch=rng.randint(1, 8),
                      field=(rng.randint(4, 30), rng.randint(4, 30)),
                      kernel=k, ci=rng.choice([3, 16, 32, 64, 96, 128, 256]),
                      co=8 * rng.randint(1, 32),
                      groups=rng.choice([1, 1, 1, 2]), padLower=lo,
                      padUpper=hi)
            if rng.random() < 0.4:
                kw["stride"] = (rng.randint(1, 3), rng.randint(1, 3))
            if rng.random() < 0.2:
                kw["idil"] = (rng.randint(1, 2), rng.randint(1, 2))
            if rng.random() < 0.2:
                kw["kdil"] = (rng.randint(1, 2), rng.randint(1, 2))
        dtype = rng.choice([pa.HALF, pa.HALF, pa.FLOAT])
        try:
            p = make_params(dtype, pa.FLOAT, **kw)
            plan = pa.Plan(p)
        except pa.MxconvError:
            continue  # no valid convolution (kernel larger than the field)
        line = [l for l in plan.describe().splitlines()
                if l.strip().startswith("kernel ")][0]
        print("case", case, kind, kw, dtype, line.strip(), flush=True)
        _exact(oracle, p, None, 7000 + case)
        kernels[line.split(None, 1)[1].split(",")[0].split("(")[0].strip()] += 1
    # every family of kernels took part
    assert len(kernels) >= 3, kernels
    print(dict(kernels))


def test_weight_deltas_random_dense_layers(oracle):
    from test_weight_update import DENSE_WU, run_weight_update
    rng = random.Random(20250613)
    dense = other = 0
    for case in range(400):
        field = tuple(rng.randint(2, 24)
                      for _ in range(rng.choice([1, 2, 2, 2])))
        kernel = tuple(rng.randint(1, min(5, f)) for f in field)
        lo, hi = _pads(rng, field, 3)
        kw = dict(batch=rng.randint(1, 40), field=field, kernel=kernel,
                  ci=8 * rng.randint(2, 20), co=8 * rng.randint(2, 36),
                  groups=rng.choice([1, 1, 1, 2, 3]), padLower=lo,
                  padUpper=hi)
        if rng.random() < 0.15:
            kw["itl"] = tuple(rng.randint(0, 1) for _ in field)
        if rng.random() < 0.15:
            kw["itu"] = tuple(rng.randint(0, 1) for _ in field)
        try:
            p = make_params(pa.HALF, pa.FLOAT, **kw)
            plan = pa.WeightUpdatePlan(p)
        except pa.MxconvError:
            continue
        is_dense = DENSE_WU in plan.describe()
        if not is_dense and rng.random() < 0.8:
            continue  # (mostly the dense kernel; some of the pass's own path)
        print("case", case, kw, "dense" if is_dense else "other", flush=True)
        r = np.random.default_rng(5000 + case)
        G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                     p.outputChannelsPerConvGroup)
        x = r.choice([-1.0, 1.0], (p.batchSize, G * Ci, *p.inputFieldShape))
        dz = r.choice([-1.0, 1.0],
                      (p.batchSize, G * Co, *p.getOutputFieldShape()))
        got, _ = run_weight_update(p, x.astype(np.float16),
                                   dz.astype(np.float16))
        np.testing.assert_array_equal(
            got, oracle.weight_deltas(p, x, dz, threads=8))
        dense += is_dense
        other += not is_dense
    assert dense >= 40 and other >= 20, (dense, other)


def test_depthwise_row_rings_random_layers(oracle):
    """The persistent depthwise kernels (forward 3x3 and 5x5, weight deltas
    3x3), forced onto random layers: strips and bands of every raggedness."""
    from test_weight_update import run_weight_update
    rng = random.Random(20250614)
    options = {"planConstraints": json.dumps({"gfx950": {"rowRing": 1}})}
    fwd = wu = 0
    for case in range(160):
        s = rng.choice([1, 2])
        lo, hi = _pads(rng, (0, 0), 2)
        k = 5 if case % 3 == 2 else 3
        kw = dict(batch=rng.randint(1, 9),
                  field=(rng.randint(3, 45), rng.randint(3, 90)),
                  kernel=(k, k), ci=1, co=1,
                  groups=8 * (rng.randint(1, 28) if case % 4
                              else rng.randint(29, 256)),
                  padLower=lo, padUpper=hi, stride=(s, s))
        if rng.random() < 0.15:
            kw["itl"] = (rng.randint(0, 1), rng.randint(0, 1))
        try:
            p = make_params(pa.HALF, pa.FLOAT, **kw)
            plan = pa.Plan(p, options)
        except pa.MxconvError:
            continue  # no valid convolution
        if "depthwise direct" not in plan.describe():
            continue  # (too small a layer for the depthwise kernels)
        print("case", case, kw, flush=True)
        assert "LDS ring" in plan.describe(), plan.describe()
        _exact(oracle, p, options, 9000 + case)
        fwd += 1
        if case % 2 or k == 5:
            continue  # (the weight-delta kernel takes 3 x 3 taps)
        r = np.random.default_rng(9500 + case)
        C = p.numConvGroups
        x = r.choice([-1.0, 1.0], (p.batchSize, C, *p.inputFieldShape))
        dz = r.choice([-1.0, 1.0], (p.batchSize, C, *p.getOutputFieldShape()))
        got, wplan = run_weight_update(p, x.astype(np.float16),
                                       dz.astype(np.float16), options=options)
        assert "LDS rings" in wplan.describe(), wplan.describe()
        np.testing.assert_array_equal(
            got, oracle.weight_deltas(p, x, dz, threads=8))
        wu += 1
    assert fwd >= 100 and wu >= 40, (fwd, wu)

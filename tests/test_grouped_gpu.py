"""Conv groups run as one by the matrix-core kernels (the planner's
convGroupsPerGroup): layers of many groups of a few channels, against the CPU
oracle through the C ABI.  +-1 data with fp32 output: exact (the block-diagonal
weights' zeros add nothing); half output: relative L2 <= 1e-3; fp8 <= 1e-3."""
import json

import numpy as np
import pytest

import poplibs_amd as pa
from helpers import make_params, random_data, rel_l2

pytestmark = pytest.mark.gpu
FUSED = "conv groups per group"


def _opts(per_group=None, **gfx):
    doc = {}
    if per_group is not None:
        doc["convGroupsPerGroup"] = per_group
    if gfx:
        doc["gfx950"] = gfx
    return {"planConstraints": json.dumps(doc)} if doc else None


def _run(oracle, p, seed, tol, options=None, bias=True, expect=None):
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
    text = plan.describe()
    if expect is not None:
        assert ("%s      %d " % (FUSED, expect) in text) == (expect > 1), text
    want = oracle.convolution(p, ad, wd, bd if bias else None, threads=8)
    if tol == 0:
        np.testing.assert_array_equal(got, want)
    else:
        assert rel_l2(got, want) <= tol
    return plan


# (parameters, groups the planner takes as one)
CASES = [
    # ResNeXt-like: 32 groups of 4 / 8 channels, 3x3
    (dict(batch=2, field=(14, 15), kernel=(3, 3), ci=4, co=4, groups=32,
          pad=1), 16),
    (dict(batch=2, field=(9, 11), kernel=(3, 3), ci=8, co=8, groups=32,
          pad=1), 8),
    # strided, more output than input channels, groups that do not all fit
    # one fused group evenly: 12 groups of 16 -> 24, four as one
    (dict(batch=3, field=(13, 9), kernel=(3, 3), ci=16, co=24, groups=12,
          pad=1, stride=2), 4),
    # 1x1 (the pointwise kernel takes the fused layer), 2 channels per group
    (dict(batch=2, field=(12, 12), kernel=(1, 1), ci=2, co=2, groups=64), 32),
    # 24 channels per group: three groups make 72 channels = nine vectors
    (dict(batch=2, field=(10, 7), kernel=(3, 3), ci=24, co=24, groups=6,
          pad=1), 3),
    # a 1-D field, kernel dilation
    (dict(batch=2, field=(40,), kernel=(3,), ci=8, co=4, groups=16, pad=2,
          kdil=2), 8),
    # a depthwise layer with a channel multiplier: 64 groups of 1 -> 2
    (dict(batch=2, field=(10, 9), kernel=(3, 3), ci=1, co=2, groups=64,
          pad=1), 64),
    # left alone: groups of 32 channels, depthwise, many outputs per group
    (dict(batch=2, field=(9, 9), kernel=(3, 3), ci=32, co=32, groups=4,
          pad=1), 1),
    (dict(batch=2, field=(9, 9), kernel=(3, 3), ci=4, co=64, groups=8,
          pad=1), 1),
]


@pytest.mark.parametrize("kw,expect", CASES)
@pytest.mark.parametrize("out_type", [pa.FLOAT, pa.HALF])
def test_grouped_layers_match_oracle(oracle, kw, expect, out_type):
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    _run(oracle, p, 41, 0 if out_type == pa.FLOAT else 1e-3, expect=expect)


@pytest.mark.parametrize("per_group", [1, 2, 4, 8, 32])
def test_grouped_constraint_is_taken(oracle, per_group):
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(9, 10), kernel=(3, 3),
                    ci=8, co=8, groups=32, pad=1)
    plan = _run(oracle, p, 42, 0, options=_opts(per_group), expect=per_group)
    # the plan's own constraints give the same plan back
    from test_plan_constraints_dump import _tiling
    again = pa.Plan(p, {"planConstraints": plan.constraints()})
    assert _tiling(again) == _tiling(plan)
    assert again.packs_like(plan)


def test_grouped_constraint_that_cannot_be_taken_means_by_itself(oracle):
    # 5 does not divide 32 groups; 4 groups of 3 channels are no whole vector
    p = make_params(pa.HALF, pa.FLOAT, batch=1, field=(6, 6), kernel=(3, 3),
                    ci=8, co=8, groups=32, pad=1)
    assert FUSED not in pa.Plan(p, _opts(5)).describe()
    p = make_params(pa.HALF, pa.FLOAT, batch=1, field=(6, 6), kernel=(3, 3),
                    ci=3, co=3, groups=8, pad=1)
    _run(oracle, p, 43, 0, options=_opts(4), expect=1)


@pytest.mark.parametrize("gfx", [dict(patch=2), dict(patch=0, blockN=128),
                                 dict(patch=0, splitK=2)])
def test_grouped_through_each_matrix_core_tiling(oracle, gfx):
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(14, 14), kernel=(3, 3),
                    ci=8, co=16, groups=16, pad=1)
    _run(oracle, p, 44, 0, options=_opts(8, **gfx), expect=8)


def test_grouped_fp8(oracle):
    from test_fast_gpu import _fp8_case
    p = make_params(pa.QUARTER, pa.HALF, batch=2, field=(9, 9), kernel=(3, 3),
                    ci=16, co=16, groups=16, pad=1)
    got, want, plan = _fp8_case(oracle, p, 45, 1, 0)
    assert FUSED + "      8 " in plan.describe(), plan.describe()
    assert rel_l2(got, want) <= 1e-3


def test_grouped_backward_pass(oracle):
    """The gradient parameters of a grouped layer are grouped alike: the
    backward pass takes the same route."""
    from gpu_helpers import quantize, run_conv
    from test_backward import transpose_chans_flip
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(9, 8), kernel=(3, 3),
                    ci=4, co=8, groups=32, pad=1)
    rng = np.random.default_rng(46)
    out_shape = (p.batchSize, p.getNumOutputChans(), *p.getOutputFieldShape())
    dz = rng.choice([-1.0, 1.0], size=out_shape)
    w = rng.choice([-1.0, 1.0], size=(32, 8, 4, 3, 3))
    bwd = pa.getGradientParams(p)
    options = {"pass": "TRAINING_BWD"}
    got, plan = run_conv(bwd, quantize(dz, pa.HALF)[0],
                         quantize(transpose_chans_flip(w, 2), pa.HALF)[0],
                         None, options, return_plan=True)
    assert FUSED in plan.describe(), plan.describe()
    want = oracle.convolution_backward(p, dz, w, threads=8)
    np.testing.assert_array_equal(got, want)


WU_CASES = [
    # (layer, groups taken as one)
    (dict(batch=4, field=(9, 8), kernel=(3, 3), ci=4, co=4, groups=32,
          pad=1), 16),
    (dict(batch=3, field=(12, 12), kernel=(3, 3), ci=8, co=16, groups=16,
          pad=1, stride=2), 8),
    (dict(batch=2, field=(10, 10), kernel=(1, 1), ci=16, co=8, groups=8), 4),
    (dict(batch=4, field=(9, 8), kernel=(3, 3), ci=32, co=32, groups=4,
          pad=1), 1),
    (dict(batch=3, field=(8, 8), kernel=(3, 3), ci=1, co=2, groups=64,
          pad=1), 64),
]


@pytest.mark.parametrize("kw,expect", WU_CASES)
@pytest.mark.parametrize("weight_deltas", [None, 0, 1])
def test_grouped_weight_deltas(oracle, kw, expect, weight_deltas):
    """The pass is planned for the layer with the groups taken as one and
    hands back the diagonal blocks: +-1 tensors, exact.  Through the planner's
    choice of kernel, the pass's own convolution (0) and the kernel that
    reads the layer's tensors as they are (1)."""
    from test_weight_update import run_weight_update
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, weight_deltas, flush=True)
    rng = np.random.default_rng(47)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    x = rng.choice([-1.0, 1.0], (p.batchSize, G * Ci, *p.inputFieldShape))
    dz = rng.choice([-1.0, 1.0],
                    (p.batchSize, G * Co, *p.getOutputFieldShape()))
    options = None if weight_deltas is None else _opts(
        None, weightDeltas=weight_deltas)
    got, plan = run_weight_update(p, x.astype(np.float16),
                                  dz.astype(np.float16), options)
    assert ("%s      %d (the weight update" % (FUSED, expect)
            in plan.describe()) == (expect > 1), plan.describe()
    np.testing.assert_array_equal(got, oracle.weight_deltas(p, x, dz,
                                                            threads=8))


def test_grouped_weight_update_in_place(oracle):
    from test_weight_update import run_weight_update
    p = make_params(pa.HALF, pa.HALF, batch=2, field=(8, 7), kernel=(3, 3),
                    ci=4, co=8, groups=32, pad=1)
    rng = np.random.default_rng(48)
    x = rng.choice([-1.0, 1.0], (2, 32 * 4, 8, 7))
    dz = rng.choice([-1.0, 1.0], (2, 32 * 8, 8, 7))
    w = rng.integers(-3, 4, (32, 8, 4, 3, 3)).astype(np.float64)
    got, plan = run_weight_update(p, x.astype(np.float16),
                                  dz.astype(np.float16), None,
                                  w.astype(np.float16), -0.25)
    assert FUSED in plan.describe()
    np.testing.assert_array_equal(
        got, w - 0.25 * oracle.weight_deltas(p, x, dz, threads=8))

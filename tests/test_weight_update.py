"""Weight update pass: the gradient with respect to the forward weights,
computed as the reference does - a forward convolution with
getWeightUpdateParams (lib/poplin/Convolution.cpp:3390-3435) on activations
and deltas with batch and channel axes exchanged (:3437-3483) - and checked
against a restatement of poplibs_test::conv::weightUpdate
(lib/poplibs_test/Convolution.cpp:724-898).

What pins the weight update oracle without running reference code:
  * ordinary parameters: torch autograd of conv1d/2d/3d in float64;
  * every transform: the forward pass is linear in its weights, so
    <conv(x, w), dz> == <w, weightDeltas(x, dz)> for any w, with the forward
    oracle pinned elsewhere;
and getWeightUpdateParams by the identity the reference relies on:
  convolution(getWeightUpdateParams(p), swap(x), swap(dz)) == swap(dW).
"""
import random

import numpy as np
import pytest
import torch

import poplibs_amd as pa
from helpers import make_params, random_params, rel_l2

from test_backward import TORCH_CASES


@pytest.mark.parametrize("kw", TORCH_CASES)
def test_oracle_weight_deltas_match_torch_autograd(oracle, kw):
    p = make_params(pa.FLOAT, **kw)
    nd = len(p.inputFieldShape)
    rng = np.random.default_rng(4)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    x = rng.standard_normal((p.batchSize, G * Ci, *p.inputFieldShape))
    w = rng.standard_normal((G, Co, Ci, *p.kernelShape))
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    pads = []
    for d in reversed(range(nd)):
        pads += [it.paddingLower[d], it.paddingUpper[d]]
    xp = torch.nn.functional.pad(torch.tensor(x), pads)
    wt = torch.tensor(w.reshape(G * Co, Ci, *p.kernelShape),
                      requires_grad=True)
    bias = torch.zeros(G * Co, dtype=torch.float64, requires_grad=True)
    conv = {1: torch.nn.functional.conv1d, 2: torch.nn.functional.conv2d,
            3: torch.nn.functional.conv3d}[nd]
    y = conv(xp, wt, bias, stride=tuple(ot.stride),
             dilation=tuple(kt.dilation), groups=G)
    dz = rng.standard_normal(tuple(y.shape))
    y.backward(torch.tensor(dz))
    dw, db = oracle.weight_deltas(p, x, dz, threads=3, with_bias=True)
    np.testing.assert_allclose(
        dw, wt.grad.numpy().reshape(G, Co, Ci, *p.kernelShape), atol=1e-11)
    np.testing.assert_allclose(db, bias.grad.numpy(), atol=1e-11)
    # the reference's model applies them as a gradient-descent step
    w2, b2 = oracle.weight_update(p, 0.25, x, dz, w, np.ones(G * Co))
    np.testing.assert_allclose(w2, w - 0.25 * dw, atol=1e-12)
    np.testing.assert_allclose(b2, 1 - 0.25 * db, atol=1e-12)


def _random_case(r, rng):
    p = random_params(r)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    x = rng.standard_normal((p.batchSize, G * Ci, *p.inputFieldShape))
    w = rng.standard_normal((G, Co, Ci, *p.kernelShape))
    dz = rng.standard_normal((p.batchSize, G * Co, *p.getOutputFieldShape()))
    return p, x, w, dz


def test_oracle_weight_deltas_are_the_adjoint_in_the_weights(oracle):
    r, rng = random.Random(13), np.random.default_rng(13)
    for _ in range(150):
        p, x, w, dz = _random_case(r, rng)
        lhs = np.vdot(oracle.convolution(p, x, w), dz)
        rhs = np.vdot(w, oracle.weight_deltas(p, x, dz))
        assert abs(lhs - rhs) <= 1e-9 * (1 + abs(lhs)), p


def wu_operands(p, x, dz):
    """Forward activations and deltas -> the weight update convolution's
    activations [Ci][G*B][field] and weights [G][Co][B][outField]
    (lib/poplin/Convolution.cpp:3459-3472)."""
    G, Ci, Co, B = (p.numConvGroups, p.inputChannelsPerConvGroup,
                    p.outputChannelsPerConvGroup, p.batchSize)
    field, out_field = tuple(p.inputFieldShape), tuple(p.getOutputFieldShape())
    acts = x.reshape(B, G, Ci, *field)
    acts = np.moveaxis(acts, (0, 1, 2), (2, 1, 0)).reshape(Ci, G * B, *field)
    weights = dz.reshape(B, G, Co, *out_field)
    weights = np.moveaxis(weights, (0, 1, 2), (2, 0, 1))
    return np.ascontiguousarray(acts), np.ascontiguousarray(weights)


def wu_result_to_weights(p, out):
    """The weight update convolution's output [Ci][G*Co][kernel] -> weight
    deltas [G][Co][Ci][kernel] (:3478-3482)."""
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    out = out.reshape(Ci, G, Co, *p.kernelShape)
    return np.ascontiguousarray(np.moveaxis(out, (0, 1, 2), (2, 0, 1)))


def test_weight_update_params_identity_and_canonical_form(oracle):
    r, rng = random.Random(14), np.random.default_rng(14)
    for _ in range(150):
        p, x, _, dz = _random_case(r, rng)
        wp = pa.getWeightUpdateParams(p)
        assert wp == wp.canonicalize()
        assert wp.getOutputFieldShape() == list(p.kernelShape)
        assert wp.kernelShape == list(p.getOutputFieldShape())
        assert wp.batchSize == p.inputChannelsPerConvGroup
        assert wp.inputChannelsPerConvGroup == p.batchSize
        assert wp.outputChannelsPerConvGroup == p.outputChannelsPerConvGroup
        want = oracle.weight_deltas(p, x, dz)
        acts, weights = wu_operands(p, x, dz)
        got = wu_result_to_weights(p, oracle.convolution(wp, acts, weights))
        np.testing.assert_allclose(got, want, atol=1e-10)


def test_weight_update_params_known_answer():
    # 3x3, stride 2, pad 1 on 8x8 -> 4x4: the deltas become a 4x4 kernel
    # dilated by the stride, sliding over the padded activations with the
    # forward kernel dilation (1) as stride; the last padding row is never
    # reached, so the pass truncates it.
    p = make_params(pa.HALF, batch=4, field=(8, 8), kernel=(3, 3), ci=16,
                    co=32, stride=2, pad=1)
    wp = pa.getWeightUpdateParams(p)
    assert wp.batchSize == 16 and wp.inputChannelsPerConvGroup == 4
    assert wp.outputChannelsPerConvGroup == 32
    assert wp.inputFieldShape == [8, 8] and wp.kernelShape == [4, 4]
    assert wp.kernelTransform.dilation == [2, 2]
    assert wp.inputTransform.paddingLower == [1, 1]
    assert wp.inputTransform.paddingUpper == [0, 0]
    assert wp.outputTransform.stride == [1, 1]
    assert wp.getOutputFieldShape() == [3, 3]


# ---------------------------------------------------------------------------
# GPU: the same pass through the C ABI.

def run_weight_update(p, x_q, dz_q, options=None, weights_q=None, scale=None):
    """x_q [B][G*Ci][field...], dz_q [B][G*Co][outField...] in the device
    element type, external layout.  Returns the weight deltas (or, with
    weights_q and scale, the updated weights) as float64 and the plan."""
    from gpu_helpers import _TORCH_DTYPE, device
    nd = len(p.inputFieldShape)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    plan = pa.WeightUpdatePlan(p, options)
    # channels-last device tensors
    to_cl = (0, *range(2, 2 + nd), 1)
    x = device(np.ascontiguousarray(x_q.transpose(to_cl)), p.inputType)
    dz = device(np.ascontiguousarray(dz_q.transpose(to_cl)), p.inputType)
    ws_bytes = plan.workspace_bytes()
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    if weights_q is None:
        out = torch.empty((G, Co, Ci, *p.kernelShape),
                          dtype=_TORCH_DTYPE[p.outputType], device="cuda:0")
        plan.calculate_weight_deltas(dz.data_ptr(), x.data_ptr(),
                                     out.data_ptr(), ws.data_ptr(), ws_bytes,
                                     stream)
    else:
        out = device(weights_q, p.inputType)
        plan.weight_update(dz.data_ptr(), out.data_ptr(), x.data_ptr(), scale,
                           ws.data_ptr(), ws_bytes, stream)
    torch.cuda.synchronize()
    return out.cpu().numpy().astype(np.float64), plan


WU_GPU_CASES = [
    dict(batch=4, field=(14, 14), kernel=(3, 3), ci=32, co=48, pad=1),
    dict(batch=2, field=(9, 9), kernel=(1, 1), ci=40, co=24),
    dict(batch=3, field=(9, 10), kernel=(3, 3), ci=8, co=16, stride=2, pad=1),
    dict(batch=2, field=(12, 13), kernel=(3, 3), groups=16, pad=1),
    dict(batch=5, field=(17,), kernel=(3,), ci=8, co=8, groups=2, kdil=2,
         padLower=(2,), padUpper=(1,)),
    dict(batch=16, field=(8, 8), kernel=(3, 3), ci=64, co=64, pad=1),
    # three field dimensions: the pass's kernel is the layer's output volume
    dict(batch=8, field=(6, 7, 5), kernel=(3, 3, 3), ci=16, co=24, pad=1),
    dict(batch=8, field=(6, 8, 8), kernel=(3, 3, 3), ci=8, co=16, pad=1,
         stride=(1, 2, 2)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kw", WU_GPU_CASES)
def test_weight_deltas_on_gpu_match_oracle(oracle, kw):
    from gpu_helpers import quantize
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    rng = np.random.default_rng(22)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    xq, xd = quantize(
        rng.standard_normal((p.batchSize, G * Ci, *p.inputFieldShape)), pa.HALF)
    dq, dd = quantize(
        rng.standard_normal((p.batchSize, G * Co, *p.getOutputFieldShape()))
        * 0.1, pa.HALF)
    got, plan = run_weight_update(p, xq, dq)
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= 1e-5, (rel_l2(got, want), plan.describe())


DENSE_WU = "matrix-core weight-delta kernel on the layer's own tensors"
DENSE_WU_CASES = [
    # the ResNet-style 3x3 layer at a small batch: 9 taps x 12 chunks
    dict(batch=4, field=(28, 28), kernel=(3, 3), ci=128, co=128, pad=1),
    # channels ragged against the 128 x 128 tile, groups, pixels no multiple
    # of 64, a 3 x 2 kernel with asymmetric padding
    dict(batch=9, field=(13, 11), kernel=(3, 2), ci=72, co=40, groups=2,
         padLower=(1, 0), padUpper=(1, 1)),
    # more channels than one tile
    dict(batch=6, field=(14, 14), kernel=(3, 3), ci=136, co=264, pad=1),
    # pointwise: one tap
    dict(batch=8, field=(12, 12), kernel=(1, 1), ci=64, co=32),
    # a 5 x 5 kernel, more padding than the window needs
    dict(batch=8, field=(12, 12), kernel=(5, 5), ci=16, co=24, pad=3),
    # input truncation (negative padding)
    dict(batch=8, field=(16, 14), kernel=(3, 3), ci=32, co=32, itl=(1, 0),
         itu=(0, 2), pad=1),
    # a 1-D field, a kernel wider than 64 pixels' worth of columns is not
    # needed: rows of 40 pixels, so 64 pixels span rows and images
    dict(batch=30, field=(40,), kernel=(5,), ci=24, co=16, pad=2),
    # tiny images: 64 pixels span several of them
    dict(batch=70, field=(4, 4), kernel=(3, 3), ci=16, co=16, pad=1),
    # one image
    dict(batch=1, field=(40, 36), kernel=(3, 3), ci=16, co=48, pad=1),
    # strided layers: the 3 x 3 and 1 x 1 downsampling layers of a ResNet at
    # a small batch, odd fields, strides that differ by dimension
    # (1024 output pixels or more, or the pass stays a convolution)
    dict(batch=8, field=(28, 28), kernel=(3, 3), ci=64, co=128, pad=1,
         stride=2),
    dict(batch=20, field=(15, 13), kernel=(1, 1), ci=48, co=80, stride=2),
    dict(batch=18, field=(17, 20), kernel=(3, 2), ci=24, co=40, groups=2,
         padLower=(1, 0), padUpper=(0, 1), stride=(3, 2)),
    dict(batch=120, field=(33,), kernel=(7,), ci=16, co=16, pad=3, stride=4),
]


FORCE_DENSE_WU = {"planConstraints": '{"gfx950": {"weightDeltas": 1}}'}


@pytest.mark.gpu
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
@pytest.mark.parametrize("kw", DENSE_WU_CASES)
def test_dense_weight_deltas_from_the_layers_own_tensors(oracle, kw, out_type):
    from gpu_helpers import quantize
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    rng = np.random.default_rng(61)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    xq, xd = quantize(
        rng.standard_normal((p.batchSize, G * Ci, *p.inputFieldShape)), pa.HALF)
    dq, dd = quantize(
        rng.standard_normal((p.batchSize, G * Co, *p.getOutputFieldShape()))
        * 0.1, pa.HALF)
    # (by name: for grouped layers with few channels the planner prefers the
    # pass's own convolution)
    got, plan = run_weight_update(p, xq, dq, FORCE_DENSE_WU)
    assert DENSE_WU in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert got.shape == want.shape
    # fp32 accumulation; a half result is rounded once
    tol = 1e-5 if out_type == pa.FLOAT else 1e-3
    assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())


@pytest.mark.gpu
@pytest.mark.parametrize("kw", DENSE_WU_CASES[:3] + DENSE_WU_CASES[-4:])
def test_dense_weight_deltas_of_signs_are_exact(oracle, kw):
    # +-1 tensors: every product and every partial sum is a small integer
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    print("case", p, flush=True)
    rng = np.random.default_rng(62)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    x = rng.choice([-1.0, 1.0], (p.batchSize, G * Ci, *p.inputFieldShape))
    dz = rng.choice([-1.0, 1.0],
                    (p.batchSize, G * Co, *p.getOutputFieldShape()))
    got, plan = run_weight_update(p, x.astype(np.float16),
                                  dz.astype(np.float16), FORCE_DENSE_WU)
    assert DENSE_WU in plan.describe()
    np.testing.assert_array_equal(got, oracle.weight_deltas(p, x, dz,
                                                            threads=8))


@pytest.mark.gpu
def test_dense_weight_deltas_at_the_benchmark_layers_full_size(oracle):
    """configs[1] whole (N=32 28x28 128->128 3x3): 252 workgroups, 28 chunks
    of 896 pixels.  Against the oracle, and - independent of it - against the
    sum of the deltas of the two halves of the batch (the pass is linear in
    the pixels it sums over)."""
    from gpu_helpers import quantize
    kw = dict(field=(28, 28), kernel=(3, 3), ci=128, co=128, pad=1)
    p = make_params(pa.HALF, pa.FLOAT, batch=32, **kw)
    rng = np.random.default_rng(63)
    xq, xd = quantize(rng.standard_normal((32, 128, 28, 28)), pa.HALF)
    dq, dd = quantize(rng.standard_normal((32, 128, 28, 28)) * 0.05, pa.HALF)
    got, plan = run_weight_update(p, xq, dq)
    assert DENSE_WU in plan.describe()
    assert "28 chunks of 896 pixels = 252 workgroups" in plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert rel_l2(got, want) <= 1e-5, rel_l2(got, want)
    half = make_params(pa.HALF, pa.FLOAT, batch=16, **kw)
    lo, _ = run_weight_update(half, xq[:16], dq[:16])
    hi, _ = run_weight_update(half, xq[16:], dq[16:])
    assert rel_l2(lo + hi, got) <= 1e-6


def test_dense_weight_update_plan_choice():
    big = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3),
                      ci=128, co=128, pad=1)
    text = pa.WeightUpdatePlan(big).describe()
    assert DENSE_WU in text
    assert "9 tap x channel tiles x 28 chunks of 896 pixels = 252 workgroups" \
        in text
    # strided layers take it too
    assert DENSE_WU in pa.WeightUpdatePlan(
        make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1, stride=2)).describe()
    # dilated kernels, tiny pixel counts and fp32 tensors stay with the
    # pass's own convolution
    for kw in (dict(batch=32, field=(28, 28), kernel=(3, 3), ci=128, co=128,
                    pad=2, kdil=2),
               dict(batch=1, field=(8, 8), kernel=(3, 3), ci=128, co=128,
                    pad=1)):
        assert DENSE_WU not in pa.WeightUpdatePlan(
            make_params(pa.HALF, **kw)).describe()
    assert DENSE_WU not in pa.WeightUpdatePlan(
        make_params(pa.FLOAT, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)).describe()
    # ... and a kernel named in planConstraints is honoured
    opts = {"planConstraints": '{"gfx950": {"kernel": "igemm"}}'}
    assert DENSE_WU not in pa.WeightUpdatePlan(big, opts).describe()


@pytest.mark.gpu
def test_weight_deltas_of_a_small_batch_run_on_the_matrix_cores(oracle):
    # the pass's input channels are the layer's batch: 4 of them are padded
    # to a whole vector and the pass stays on the matrix cores
    from gpu_helpers import quantize
    p = make_params(pa.HALF, pa.FLOAT, batch=4, field=(14, 14), kernel=(3, 3),
                    ci=32, co=48, pad=1)
    rng = np.random.default_rng(26)
    xq, xd = quantize(rng.standard_normal((4, 32, 14, 14)), pa.HALF)
    dq, dd = quantize(rng.standard_normal((4, 48, 14, 14)) * 0.1, pa.HALF)
    got, plan = run_weight_update(p, xq, dq)
    assert "implicit GEMM" in plan.describe(), plan.describe()
    assert "input channels padded      4 -> 8" in plan.describe()
    assert rel_l2(got, oracle.weight_deltas(p, xd, dd, threads=8)) <= 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("co", [3, 5])
@pytest.mark.parametrize("dt", [pa.HALF, pa.FLOAT])
def test_weight_deltas_of_a_layer_with_few_output_channels(oracle, co, dt):
    # (an RGB head.)  The pass has `co` output channels, a long K (the layer's
    # field x its batch) and a handful of output tiles: K is cut into parts,
    # and the parts are added one channel per thread where the channel count
    # is no multiple of four.
    from gpu_helpers import quantize
    p = make_params(dt, pa.FLOAT, batch=8, field=(28, 28), kernel=(3, 3),
                    ci=32, co=co, pad=1)
    rng = np.random.default_rng(28)
    xq, xd = quantize(rng.standard_normal((8, 32, 28, 28)), dt)
    dq, dd = quantize(rng.standard_normal((8, co, 28, 28)) * 0.1, dt)
    got, plan = run_weight_update(p, xq, dq)
    assert "implicit GEMM" in plan.describe(), plan.describe()
    assert "K split into parts" in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert rel_l2(got, want) <= 1e-5, (rel_l2(got, want), plan.describe())


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [pa.HALF, pa.FLOAT])
@pytest.mark.parametrize("kw", [
    dict(batch=8, field=(1500,), kernel=(3,), ci=16, co=24, pad=1),
    dict(batch=5, field=(900,), kernel=(5,), ci=8, co=8, pad=2, stride=2,
         groups=2),
])
def test_weight_deltas_of_a_long_1d_layer(oracle, kw, dt):
    # the pass's own convolution has a kernel as long as the layer's output:
    # hundreds of taps in one dimension, on the matrix cores all the same
    from gpu_helpers import quantize
    p = make_params(dt, pa.FLOAT, **kw)
    rng = np.random.default_rng(29)
    xq, xd = quantize(rng.standard_normal(
        (p.batchSize, p.getNumInputChans(), *p.inputFieldShape)), dt)
    dq, dd = quantize(rng.standard_normal(
        (p.batchSize, p.getNumOutputChans(), *p.getOutputFieldShape())) * 0.1,
        dt)
    got, plan = run_weight_update(p, xq, dq)
    assert "generic direct" not in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert rel_l2(got, want) <= 1e-5, (rel_l2(got, want), plan.describe())


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [8, 16])
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_weight_deltas_of_a_truncated_kernel(oracle, batch, out_type):
    # Kernel truncation of the layer is output padding of its weight update
    # pass (the deltas of the truncated taps are zero): with a batch that is
    # a whole vector the pass runs on the matrix cores, and the padded rows
    # of the deltas have to be written all the same.
    from gpu_helpers import quantize
    p = make_params(pa.HALF, out_type, batch=batch, field=(8, 8),
                    kernel=(3, 3), ci=16, co=16, ktl=(1, 0), pad=1)
    rng = np.random.default_rng(27)
    xq, xd = quantize(rng.standard_normal((batch, 16, 8, 8)), pa.HALF)
    dq, dd = quantize(
        rng.standard_normal((batch, 16, *p.getOutputFieldShape())) * 0.1,
        pa.HALF)
    got, plan = run_weight_update(p, xq, dq)
    assert "implicit GEMM" in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert got.shape == want.shape
    assert not want[:, :, :, 0, :].any()  # the truncated kernel row
    tol = 1e-3 if out_type == pa.HALF else 1e-5
    assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())
    np.testing.assert_array_equal(got[:, :, :, 0, :], 0)


DEPTHWISE_WU_CASES = [
    dict(batch=3, field=(20, 21), kernel=(3, 3), groups=24, stride=2, pad=1),
    dict(batch=2, field=(14, 14), kernel=(5, 5), groups=16, pad=2),
    dict(batch=4, field=(11, 9), kernel=(3, 2), groups=8, kdil=(2, 1),
         padLower=(1, 0), padUpper=(2, 1), stride=(1, 2)),
    dict(batch=2, field=(30,), kernel=(7,), groups=32, stride=3, pad=3),
    dict(batch=2, field=(12, 12), kernel=(3, 3), groups=40, itl=(1, 0),
         itu=(0, 2), pad=1),
    dict(batch=70, field=(6, 6), kernel=(3, 3), groups=8, pad=1),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kw", DEPTHWISE_WU_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_depthwise_weight_deltas_on_gpu(oracle, kw, out_type):
    from gpu_helpers import quantize
    p = make_params(pa.HALF, out_type, **kw)
    rng = np.random.default_rng(24)
    C = p.numConvGroups
    xq, xd = quantize(
        rng.standard_normal((p.batchSize, C, *p.inputFieldShape)), pa.HALF)
    dq, dd = quantize(
        rng.standard_normal((p.batchSize, C, *p.getOutputFieldShape())) * 0.1,
        pa.HALF)
    got, plan = run_weight_update(p, xq, dq)
    assert "depthwise weight-delta kernel" in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert got.shape == want.shape
    tol = 1e-3 if out_type == pa.HALF else 1e-5
    assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())


@pytest.mark.gpu
@pytest.mark.parametrize("kw", DEPTHWISE_WU_CASES[:5] + [
    dict(batch=3, field=(9, 9), kernel=(3, 3), groups=12, pad=1)])
def test_depthwise_weight_deltas_fp32(oracle, kw):
    """fp32 tensors: vectors of four channels, +-1 data exact."""
    p = make_params(pa.FLOAT, pa.FLOAT, **kw)
    rng = np.random.default_rng(25)
    C = p.numConvGroups
    x = rng.choice([-1.0, 1.0], (p.batchSize, C, *p.inputFieldShape))
    dz = rng.choice([-1.0, 1.0], (p.batchSize, C, *p.getOutputFieldShape()))
    got, plan = run_weight_update(p, x.astype(np.float32),
                                  dz.astype(np.float32))
    assert "depthwise weight-delta kernel" in plan.describe(), plan.describe()
    np.testing.assert_array_equal(got, oracle.weight_deltas(p, x, dz,
                                                            threads=8))


@pytest.mark.gpu
def test_depthwise_weight_deltas_of_signs_are_exact(oracle):
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(9, 9), kernel=(3, 3),
                    groups=16, stride=2, pad=1)
    rng = np.random.default_rng(25)
    x = rng.choice([-1.0, 1.0], size=(2, 16, 9, 9))
    dz = rng.choice([-1.0, 1.0], size=(2, 16, 5, 5))
    got, _ = run_weight_update(p, x.astype(np.float16), dz.astype(np.float16))
    np.testing.assert_array_equal(got, oracle.weight_deltas(p, x, dz))


ROW_RING = {"planConstraints": '{"gfx950": {"rowRing": 1}}'}
RING_WU = "rows of both streamed through LDS rings"
RING_WU_CASES = [
    # stride 2: strips narrower than the image, bands of one row
    dict(batch=3, field=(20, 21), kernel=(3, 3), groups=24, stride=2, pad=1),
    # stride 1, asymmetric padding, several strips (28 vectors per pixel)
    dict(batch=5, field=(17, 40), kernel=(3, 3), groups=224, stride=1,
         padLower=(2, 0), padUpper=(0, 1)),
    # input truncation (negative padding), ragged last strip and band
    dict(batch=2, field=(29, 71), kernel=(3, 3), groups=40, stride=2,
         itl=(1, 0), itu=(0, 2), pad=1),
    # bands of several rows
    dict(batch=40, field=(36, 30), kernel=(3, 3), groups=16, stride=2, pad=1),
    # tiny images
    dict(batch=70, field=(3, 3), kernel=(3, 3), groups=8, pad=1),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kw", RING_WU_CASES)
@pytest.mark.parametrize("out_type", [pa.HALF, pa.FLOAT])
def test_depthwise_weight_deltas_row_rings(oracle, kw, out_type):
    from gpu_helpers import quantize
    p = make_params(pa.HALF, out_type, **kw)
    print("case", p, flush=True)
    rng = np.random.default_rng(26)
    C = p.numConvGroups
    xq, xd = quantize(
        rng.standard_normal((p.batchSize, C, *p.inputFieldShape)), pa.HALF)
    dq, dd = quantize(
        rng.standard_normal((p.batchSize, C, *p.getOutputFieldShape())) * 0.1,
        pa.HALF)
    got, plan = run_weight_update(p, xq, dq, options=ROW_RING)
    assert RING_WU in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert got.shape == want.shape
    tol = 1e-3 if out_type == pa.HALF else 1e-5
    assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())


@pytest.mark.gpu
@pytest.mark.parametrize("kw", RING_WU_CASES[:3])
def test_depthwise_weight_deltas_row_rings_of_signs_are_exact(oracle, kw):
    p = make_params(pa.HALF, pa.FLOAT, **kw)
    rng = np.random.default_rng(27)
    C = p.numConvGroups
    x = rng.choice([-1.0, 1.0], (p.batchSize, C, *p.inputFieldShape))
    dz = rng.choice([-1.0, 1.0], (p.batchSize, C, *p.getOutputFieldShape()))
    got, plan = run_weight_update(p, x.astype(np.float16),
                                  dz.astype(np.float16), options=ROW_RING)
    assert RING_WU in plan.describe()
    np.testing.assert_array_equal(got, oracle.weight_deltas(p, x, dz,
                                                            threads=8))


def test_depthwise_weight_update_row_rings_plan_choice():
    big = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                      groups=96, stride=2, pad=1)
    text = pa.WeightUpdatePlan(big).describe()
    assert RING_WU in text and "256 persistent workgroups" in text, text
    off = pa.WeightUpdatePlan(
        big, {"planConstraints": '{"gfx950": {"rowRing": 0}}'}).describe()
    assert "depthwise weight-delta kernel" in off and RING_WU not in off
    small = make_params(pa.HALF, **DEPTHWISE_WU_CASES[0])
    assert RING_WU not in pa.WeightUpdatePlan(small).describe()
    # a 5 x 5 kernel stays with the slices whatever is asked
    five = make_params(pa.HALF, **DEPTHWISE_WU_CASES[1])
    assert RING_WU not in pa.WeightUpdatePlan(five, ROW_RING).describe()


@pytest.mark.gpu
def test_weight_update_applies_scaled_deltas(oracle):
    from gpu_helpers import quantize
    p = make_params(pa.HALF, pa.HALF, batch=4, field=(10, 10), kernel=(3, 3),
                    ci=16, co=32, pad=1)
    rng = np.random.default_rng(23)
    xq, xd = quantize(rng.standard_normal((4, 16, 10, 10)), pa.HALF)
    dq, dd = quantize(rng.standard_normal((4, 32, 10, 10)) * 0.1, pa.HALF)
    wq, wd = quantize(rng.standard_normal((1, 32, 16, 3, 3)), pa.HALF)
    got, _ = run_weight_update(p, xq, dq, weights_q=wq, scale=-0.125)
    want, _ = oracle.weight_update(p, 0.125, xd, dd, wd, np.zeros(32))
    # deltas rounded to half, then the sum rounded to half
    assert rel_l2(got, want) <= 2e-3, rel_l2(got, want)
    # a float-output plan is refused: the deltas must have the weights' type
    pf = make_params(pa.HALF, pa.FLOAT, batch=4, field=(10, 10), kernel=(3, 3),
                     ci=16, co=32, pad=1)
    with pytest.raises(pa.MxconvError) as e:
        run_weight_update(pf, xq, dq, weights_q=wq, scale=1.0)
    assert e.value.status == pa.Status.INVALID_PARAMS


PRODUCT_WU = "one matrix product, transpose(deltas) x activations"
FC_CASES = [
    # (batch, input channels, output channels, field)
    (70, 96, 64, ()),
    (5, 20, 24, ()),          # channel counts that are no whole vector
    (256, 512, 136, (1,)),
    (33, 8, 1000, (1, 1)),
    (1, 64, 32, ()),          # one sample
    (300, 3, 7, ()),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dt,ot", [(pa.HALF, pa.HALF), (pa.HALF, pa.FLOAT),
                                   (pa.FLOAT, pa.FLOAT)])
@pytest.mark.parametrize("batch,ci,co,field", FC_CASES)
def test_weight_deltas_of_a_layer_without_spatial_extent(oracle, batch, ci,
                                                         co, field, dt, ot):
    # deltas[co][ci] = sum over the batch of dZ[b][co] x[b][ci]: one matrix
    # product whose result is in weight order as it is
    from gpu_helpers import quantize
    p = make_params(dt, ot, batch=batch, field=field, kernel=(1,) * len(field),
                    ci=ci, co=co)
    rng = np.random.default_rng(31)
    xq, xd = quantize(rng.standard_normal((batch, ci, *field)), dt)
    dq, dd = quantize(rng.standard_normal((batch, co, *field)) * 0.1, dt)
    got, plan = run_weight_update(p, xq, dq)
    assert PRODUCT_WU in plan.describe(), plan.describe()
    want = oracle.weight_deltas(p, xd, dd, threads=8)
    assert got.shape == want.shape
    tol = 1e-3 if ot == pa.HALF else 1e-5
    assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())
    # the pass's own convolution, by name, gives the same deltas
    own, plan0 = run_weight_update(
        p, xq, dq, {"planConstraints": '{"gfx950": {"weightDeltas": 0}}'})
    assert PRODUCT_WU not in plan0.describe()
    assert rel_l2(own, want) <= tol


@pytest.mark.gpu
def test_weight_update_of_a_fully_connected_layer(oracle):
    from gpu_helpers import quantize
    p = make_params(pa.HALF, pa.HALF, batch=48, field=(), kernel=(), ci=40,
                    co=72)
    rng = np.random.default_rng(32)
    xq, xd = quantize(rng.standard_normal((48, 40)), pa.HALF)
    dq, dd = quantize(rng.standard_normal((48, 72)) * 0.1, pa.HALF)
    wq, wd = quantize(rng.standard_normal((1, 72, 40)), pa.HALF)
    got, plan = run_weight_update(p, xq, dq, weights_q=wq, scale=-0.25)
    assert PRODUCT_WU in plan.describe()
    want, _ = oracle.weight_update(p, 0.25, xd, dd, wd, np.zeros(72))
    assert rel_l2(got, want) <= 2e-3, rel_l2(got, want)


def test_weight_deltas_as_a_product_plan_choice():
    fc = make_params(pa.HALF, batch=256, field=(), kernel=(), ci=1024, co=512)
    assert PRODUCT_WU in pa.WeightUpdatePlan(fc).describe()
    by_name = {"planConstraints": '{"gfx950": {"weightDeltas": 2}}'}
    assert PRODUCT_WU in pa.WeightUpdatePlan(fc, by_name).describe()
    # its workspace: transposed deltas, packed activations, the deltas of an
    # update
    assert pa.WeightUpdatePlan(fc).workspace_bytes() >= \
        2 * (256 * 512 + 256 * 1024 + 512 * 1024)
    # a layer with a field is not one product over the batch ...
    conv = make_params(pa.HALF, batch=8, field=(6, 6), kernel=(1, 1), ci=64,
                       co=64)
    assert PRODUCT_WU not in pa.WeightUpdatePlan(conv).describe()
    with pytest.raises(pa.MxconvError, match="weightDeltas 2"):
        pa.WeightUpdatePlan(conv, by_name)
    # ... nor are groups, and a named kernel keeps the pass's own convolution
    grouped = make_params(pa.HALF, batch=64, field=(), kernel=(), ci=32,
                          co=32, groups=4)
    assert PRODUCT_WU not in pa.WeightUpdatePlan(grouped).describe()
    named = {"planConstraints": '{"gfx950": {"kernel": "igemm"}}'}
    assert PRODUCT_WU not in pa.WeightUpdatePlan(fc, named).describe()


@pytest.mark.gpu
def test_weight_update_random_params_on_gpu(oracle):
    from gpu_helpers import quantize
    r, rng = random.Random(32), np.random.default_rng(32)
    for _ in range(25):
        p, x, _, dz = _random_case(r, rng)
        p = pa.ConvParams(pa.FLOAT, pa.FLOAT, p.batchSize, p.inputFieldShape,
                          p.kernelShape, p.inputChannelsPerConvGroup,
                          p.outputChannelsPerConvGroup, p.numConvGroups,
                          p.inputTransform, p.kernelTransform,
                          p.outputTransform)
        xq, xd = quantize(x, pa.FLOAT)
        dq, dd = quantize(dz, pa.FLOAT)
        got, plan = run_weight_update(p, xq, dq)
        want = oracle.weight_deltas(p, xd, dd)
        assert got.shape == want.shape
        if want.size:
            assert rel_l2(got, want) <= 1e-5, (rel_l2(got, want), p)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,chans,dt,bt", [
    (1, 1, pa.FLOAT, pa.FLOAT), (1000, 7, pa.HALF, pa.HALF),
    (25088, 128, pa.HALF, pa.FLOAT), (300, 200, pa.FLOAT, pa.HALF),
    (0, 5, pa.HALF, pa.HALF)])
def test_bias_update_on_gpu(rows, chans, dt, bt):
    from gpu_helpers import device, quantize
    rng = np.random.default_rng(rows + chans)
    zq, zd = quantize(rng.standard_normal((rows, chans)), dt)
    bq, bd = quantize(rng.standard_normal(chans), bt)
    z, b = device(zq, dt), device(bq, bt)
    ws_bytes = pa.bias_update_workspace_bytes(rows, chans)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda:0")
    pa.convolutionBiasUpdate(dt, z.data_ptr(), rows, chans, bt, b.data_ptr(),
                             -0.5, ws.data_ptr(), ws_bytes)
    torch.cuda.synchronize()
    want = bd - 0.5 * zd.sum(axis=0)
    got = b.cpu().numpy().astype(np.float64)
    tol = 2e-3 if bt == pa.HALF else 1e-5
    np.testing.assert_allclose(got, want, rtol=tol,
                               atol=tol * max(1.0, np.abs(want).max()))

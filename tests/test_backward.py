"""Backward-data pass: the gradient with respect to the forward input, computed
as the reference does - a forward convolution with getGradientParams
(lib/poplin/ConvUtil.cpp:728-795) on weights passed through
weightsTransposeChansFlipXY (lib/poplin/Convolution.cpp:3262-3388) - and
checked against a restatement of poplibs_test::conv::convolutionBackward
(lib/poplibs_test/Convolution.cpp:577-722).

What pins the backward oracle without running reference code:
  * ordinary parameters: torch autograd of conv1d/2d/3d in float64;
  * every transform: the backward pass is the adjoint of the forward pass,
    <conv(x), dz> == <x, convBackward(dz)>, with the forward oracle pinned
    elsewhere;
and getGradientParams by the identity the reference relies on:
  convolution(getGradientParams(p), dz, transposeFlip(w))
      == convolutionBackward(p, dz, w).
"""
import random

import numpy as np
import pytest
import torch

import poplibs_amd as pa
from helpers import make_params, random_params, rel_l2


def transpose_chans_flip(w, nd):
    """numpy statement of weightsTransposeChansFlipXY."""
    wt = np.swapaxes(w, 1, 2)
    for axis in range(3, 3 + nd):
        wt = np.flip(wt, axis=axis)
    return np.ascontiguousarray(wt)


TORCH_CASES = [
    dict(batch=2, field=(9, 8), kernel=(3, 2), ci=3, co=4, groups=2,
         stride=(2, 1), kdil=(2, 1), pad=1),
    dict(batch=1, field=(11,), kernel=(4,), ci=2, co=3, stride=3, pad=2),
    dict(batch=2, field=(5, 6, 4), kernel=(2, 3, 2), ci=2, co=2, stride=(1, 2, 1),
         padLower=(1, 0, 1), padUpper=(0, 2, 1)),
    dict(batch=3, field=(7, 7), kernel=(1, 1), ci=5, co=2),
    # stride leaves input rows untouched: their gradient is zero
    dict(batch=1, field=(8, 9), kernel=(2, 2), ci=1, co=1, stride=(3, 4)),
]


@pytest.mark.parametrize("kw", TORCH_CASES)
def test_oracle_backward_matches_torch_autograd(oracle, kw):
    p = make_params(pa.FLOAT, **kw)
    nd = len(p.inputFieldShape)
    rng = np.random.default_rng(3)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    x = rng.standard_normal((p.batchSize, G * Ci, *p.inputFieldShape))
    w = rng.standard_normal((G, Co, Ci, *p.kernelShape))
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    xt = torch.tensor(x, requires_grad=True)
    # asymmetric padding: pad explicitly, then convolve unpadded
    pads = []
    for d in reversed(range(nd)):
        pads += [it.paddingLower[d], it.paddingUpper[d]]
    xp = torch.nn.functional.pad(xt, pads)
    conv = {1: torch.nn.functional.conv1d, 2: torch.nn.functional.conv2d,
            3: torch.nn.functional.conv3d}[nd]
    y = conv(xp, torch.tensor(w.reshape(G * Co, Ci, *p.kernelShape)),
             stride=tuple(ot.stride), dilation=tuple(kt.dilation), groups=G)
    fwd = oracle.convolution(p, x, w)
    np.testing.assert_allclose(fwd, y.detach().numpy(), atol=1e-12)
    dz = rng.standard_normal(fwd.shape)
    y.backward(torch.tensor(dz))
    got = oracle.convolution_backward(p, dz, w, threads=3)
    np.testing.assert_allclose(got, xt.grad.numpy(), atol=1e-12)


def _random_case(r, rng):
    p = random_params(r)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    x = rng.standard_normal((p.batchSize, G * Ci, *p.inputFieldShape))
    w = rng.standard_normal((G, Co, Ci, *p.kernelShape))
    dz = rng.standard_normal((p.batchSize, G * Co, *p.getOutputFieldShape()))
    return p, x, w, dz


def test_oracle_backward_is_the_adjoint_of_forward(oracle):
    r, rng = random.Random(11), np.random.default_rng(11)
    for _ in range(150):
        p, x, w, dz = _random_case(r, rng)
        lhs = np.vdot(oracle.convolution(p, x, w), dz)
        rhs = np.vdot(x, oracle.convolution_backward(p, dz, w))
        assert abs(lhs - rhs) <= 1e-9 * (1 + abs(lhs)), p


def test_gradient_params_identity_and_canonical_form(oracle):
    r, rng = random.Random(12), np.random.default_rng(12)
    for _ in range(150):
        p, _, w, dz = _random_case(r, rng)
        gp = pa.getGradientParams(p)
        assert gp == gp.canonicalize()
        assert gp.getOutputFieldShape() == list(p.inputFieldShape)
        assert gp.inputChannelsPerConvGroup == p.outputChannelsPerConvGroup
        assert gp.outputChannelsPerConvGroup == p.inputChannelsPerConvGroup
        want = oracle.convolution_backward(p, dz, w)
        got = oracle.convolution(
            gp, dz, transpose_chans_flip(w, len(p.inputFieldShape)))
        np.testing.assert_allclose(got, want, atol=1e-10)


def test_gradient_params_known_answer():
    # 3x3, stride 2, pad 1 on 8x8 -> 4x4.  Backwards: the deltas are dilated
    # by the stride and padded by kernel size - 1 minus the forward padding;
    # the forward pass never used its last padding row, so the backward pass
    # pads one more on that side (8 = 1 + (4-1)*2+1 + 2 - 3 + 1).
    p = make_params(pa.HALF, batch=4, field=(8, 8), kernel=(3, 3), ci=16,
                    co=32, stride=2, pad=1)
    gp = pa.getGradientParams(p)
    assert gp.inputFieldShape == [4, 4] and gp.kernelShape == [3, 3]
    assert gp.inputChannelsPerConvGroup == 32
    assert gp.outputChannelsPerConvGroup == 16
    assert gp.inputTransform.dilation == [2, 2]
    assert gp.inputTransform.paddingLower == [1, 1]
    assert gp.inputTransform.paddingUpper == [2, 2]
    assert gp.outputTransform.stride == [1, 1]
    assert gp.getOutputFieldShape() == [8, 8]


# ---------------------------------------------------------------------------
# GPU: the same pass through the C ABI.

BWD_GPU_CASES = [
    # forward 3x3 s1 p1, 128 -> 128: backward is again a matrix-core conv
    (dict(batch=2, field=(14, 14), kernel=(3, 3), ci=128, co=128, pad=1),
     "implicit GEMM"),
    # forward 1x1 256 -> 64: backward is the pointwise kernel's 64 -> 256?
    # (64 input channels: the big-tile kernel)
    (dict(batch=2, field=(9, 9), kernel=(1, 1), ci=256, co=64),
     "implicit GEMM"),
    # forward stride 2: the deltas are dilated going backwards - the matrix
    # cores take it as one convolution per phase of the stuffed zeros
    (dict(batch=2, field=(9, 10), kernel=(3, 3), ci=8, co=16, stride=2, pad=1),
     "4 phases"),
    # ... also a strided 1x1 shortcut, three of whose four phases are zeros
    (dict(batch=2, field=(9, 10), kernel=(1, 1), ci=16, co=24, stride=2),
     "4 phases"),
    # depthwise 3x3 stride 2: dilated deltas, one thread per output vector
    (dict(batch=2, field=(13, 12), kernel=(3, 3), groups=24, stride=2, pad=1),
     "dilated input"),
    (dict(batch=2, field=(17,), kernel=(5,), groups=8, stride=3, pad=2),
     "dilated input"),
    # ... stride 2 with 3x3 or 5x5 taps: a thread per 2x2 block of outputs.
    # No padding, even and odd fields, a channel count that is no power of
    # two, asymmetric padding, more rows than one thread's strip, 5x5
    (dict(batch=2, field=(13, 11), kernel=(3, 3), groups=8, stride=2),
     "dilated input"),
    (dict(batch=3, field=(14, 14), kernel=(3, 3), groups=40, stride=2, pad=1),
     "dilated input"),
    (dict(batch=1, field=(37, 12), kernel=(3, 3), groups=16, stride=2,
          padLower=(0, 1), padUpper=(1, 0)), "dilated input"),
    (dict(batch=2, field=(15, 14), kernel=(5, 5), groups=16, stride=2, pad=2),
     "dilated input"),
    (dict(batch=1, field=(10, 21), kernel=(5, 5), groups=8, stride=2,
          padLower=(1, 2), padUpper=(2, 0)), "dilated input"),
    # ... the forward output was padded: those deltas are cut off again
    (dict(batch=2, field=(13, 12), kernel=(3, 3), groups=16, stride=2, pad=1,
          opl=(1, 0), opu=(0, 2)), "dilated input"),
    # depthwise 3x3 stride 1 stays depthwise
    (dict(batch=2, field=(12, 13), kernel=(3, 3), groups=16, pad=1),
     "depthwise direct"),
    # groups, asymmetric padding, kernel dilation, 1-D
    (dict(batch=3, field=(17,), kernel=(3,), ci=8, co=8, groups=2, kdil=2,
          padLower=(2,), padUpper=(1,)), "implicit GEMM"),
]


@pytest.mark.gpu
@pytest.mark.parametrize("kw,kernel", BWD_GPU_CASES)
def test_backward_pass_on_gpu_matches_oracle(oracle, kw, kernel):
    from gpu_helpers import device, quantize, run_conv
    p = make_params(pa.HALF, **kw)
    nd = len(p.inputFieldShape)
    rng = np.random.default_rng(21)
    G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                 p.outputChannelsPerConvGroup)
    w = rng.standard_normal((G, Co, Ci, *p.kernelShape)) * 0.1
    dz = rng.standard_normal((p.batchSize, G * Co, *p.getOutputFieldShape()))
    wq, wd = quantize(w, pa.HALF)
    dq, dd = quantize(dz, pa.HALF)
    # weightsTransposeChansFlipXY on the device, bit-exact against numpy
    w_dev = device(wq, pa.HALF)
    wt_dev = torch.empty((G, Ci, Co, *p.kernelShape), dtype=torch.float16,
                         device="cuda:0")
    pa.weightsTransposeChansFlipXY(p, w_dev.data_ptr(), wt_dev.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    wt = wt_dev.cpu().numpy()
    np.testing.assert_array_equal(wt, transpose_chans_flip(wq, nd))
    gp = pa.getGradientParams(p)
    got, plan = run_conv(gp, dq, wt, return_plan=True)
    assert kernel in plan.describe(), plan.describe()
    want = oracle.convolution_backward(p, dd, wd, threads=8)
    assert got.shape == want.shape
    assert rel_l2(got, want) <= 1e-3, (rel_l2(got, want), p)


@pytest.mark.gpu
def test_backward_pass_random_params_on_gpu(oracle):
    from gpu_helpers import quantize, run_conv
    r, rng = random.Random(31), np.random.default_rng(31)
    for _ in range(25):
        p, _, w, dz = _random_case(r, rng)
        p = pa.ConvParams(pa.FLOAT, pa.FLOAT, p.batchSize, p.inputFieldShape,
                          p.kernelShape, p.inputChannelsPerConvGroup,
                          p.outputChannelsPerConvGroup, p.numConvGroups,
                          p.inputTransform, p.kernelTransform,
                          p.outputTransform)
        wq, wd = quantize(w, pa.FLOAT)
        dq, dd = quantize(dz, pa.FLOAT)
        gp = pa.getGradientParams(p)
        got = run_conv(gp, dq, transpose_chans_flip(wq,
                                                    len(p.inputFieldShape)))
        want = oracle.convolution_backward(p, dd, wd)
        assert got.shape == want.shape
        if want.size:
            assert rel_l2(got, want) <= 1e-5, (rel_l2(got, want), p)

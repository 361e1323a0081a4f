"""Matrix multiplication through the convolution path, as the reference does it
(lib/poplin/MatMul.cpp:236-272 getConvParams, :345-400 matMulImpl): C[g] = A[g]
* B[g] is the convolution with batch m, a 1-element field and kernel, k input
and n output channels per group, on weights transpose(B).

The checker is numpy's float64 matmul on the values the device holds; the
mapping itself is pinned on the CPU by running the convolution oracle on the
mapped operands and comparing with numpy.
"""
import numpy as np
import pytest

import poplibs_amd as pa
from poplibs_amd import capi
from helpers import rel_l2


def conv_operands(A, B):
    """A [g][m][k], B [g][k][n] -> the convolution's activations
    [m][g*k][1] and weights [g][n][k][1]."""
    g, m, k = A.shape
    acts = np.ascontiguousarray(A.transpose(1, 0, 2)).reshape(m, g * k, 1)
    weights = np.ascontiguousarray(B.transpose(0, 2, 1))[..., None]
    return acts, weights


@pytest.mark.parametrize("g,m,k,n", [(1, 5, 3, 4), (3, 4, 7, 2), (2, 1, 9, 1),
                                     (1, 5, 0, 4), (1, 0, 3, 4), (2, 3, 2, 0)])
def test_matmul_params_map_to_the_convolution(oracle, g, m, k, n):
    p = pa.matMulParams(pa.HALF, pa.FLOAT, g, m, k, n)
    assert p == pa.ConvParams(pa.HALF, pa.FLOAT, m, [1], [1], k, n, g)
    assert p.getOutputFieldShape() == [1]
    assert p.getNumberOfMACs() == g * m * k * n
    rng = np.random.default_rng(5)
    A = rng.standard_normal((g, m, k))
    B = rng.standard_normal((g, k, n))
    acts, weights = conv_operands(A, B)
    out = oracle.convolution(p, acts, weights)          # [m][g*n][1]
    C = out.reshape(m, g, n).transpose(1, 0, 2)
    np.testing.assert_allclose(C, A @ B, atol=1e-12)


def test_matmul_params_reject_bad_types():
    with pytest.raises(pa.MxconvError) as e:
        pa.matMulParams(7, pa.FLOAT, 1, 2, 2, 2)
    assert e.value.status == pa.Status.INVALID_PARAMS


def test_matmul_options():
    # every key of MatMulOptions (lib/poplin/MatMul.cpp:116-160)
    pa.matMulValidateOptions({
        "partialsType": "half", "fullyConnectedPass": "TRAINING_BWD",
        "inputRHSIsPreArranged": "true", "use128BitConvUnitLoad": "false",
        "enableMultiStageReduce": "false", "enableFastReduce": "true",
        "remapOutputTensor": "false", "availableMemoryProportion": "0.3",
        "planConstraints": "{}", "gatherOutput": "true",
        "disableSRForAMPVertices": "true"})
    pa.matMulValidateOptions({})
    for bad in ({"pass": "NONE"},                     # a convolution key
                {"partialsType": "quarter"},
                {"fullyConnectedPass": "FC_TRAINING_FWD"},
                {"enableFastReduce": "1"},
                {"availableMemoryProportion": "lots"},
                {"availableMemoryProportion": "-1"},
                {"planConstraints": "{not json"}):
        with pytest.raises(pa.MxconvError) as e:
            pa.matMulValidateOptions(bad)
        assert e.value.status == pa.Status.INVALID_OPTION, bad


PLAN_CASES = [
    # (type, g, m, k, n, options, text expected in the plan description)
    (pa.HALF, 1, 1024, 512, 512, None, "implicit GEMM"),
    (pa.HALF, 1, 4096, 256, 64, None, "pointwise streaming"),
    (pa.HALF, 1, 7, 5, 3, None, "generic direct"),
    (pa.FLOAT, 1, 64, 64, 64, None, "implicit GEMM (MFMA, fp32"),
    (pa.FLOAT, 1, 64, 62, 64, None, "generic direct"),
    (pa.FLOAT, 1, 256, 62, 256, None, "input channels padded      62 -> 64"),
    (pa.HALF, 1, 64, 64, 64,
     {"planConstraints": '{"gfx950": {"kernel": "generic"}}'}, "generic direct"),
    (pa.HALF, 4, 256, 64, 64, None, "implicit GEMM"),
]


@pytest.mark.parametrize("t,g,m,k,n,options,text", PLAN_CASES)
def test_matmul_plan_kernels(t, g, m, k, n, options, text):
    plan = pa.MatMulPlan(t, t, g, m, k, n, options)
    assert text in plan.describe(), plan.describe()
    # the plan is the one the mapped convolution gets with the mapped options
    conv = pa.Plan(pa.matMulParams(t, t, g, m, k, n),
                   dict(options or {}, **{"pass": "NONE_MATMUL"}))
    assert plan.describe() == conv.describe()
    assert plan.buffer_bytes(capi.BUF_INPUT) == g * m * k * capi.TYPE_BYTES[t]
    assert plan.buffer_bytes(capi.BUF_OUTPUT) == g * m * n * capi.TYPE_BYTES[t]


def test_matrix_entries_refuse_other_plans():
    plan = pa.Plan(pa.ConvParams(pa.HALF, pa.HALF, 1, [4], [3], 8, 8, 1))
    for call in (plan_call for plan_call in (
            capi.lib().mxconv_matmul_pack_rhs,
            capi.lib().mxconv_matmul_lhs_to_internal,
            capi.lib().mxconv_matmul_out_to_external)):
        assert call(plan._h, 16, 32, None) == pa.Status.INVALID_PARAMS


# ---------------------------------------------------------------------------
# GPU

def run_matmul(A_q, B_q, in_type, out_type, options=None, return_plan=False):
    """A_q [g][m][k], B_q [g][k][n] in the device element type -> C as float64
    and optionally the plan."""
    import torch
    from gpu_helpers import _TORCH_DTYPE, device
    g, m, k = A_q.shape
    n = B_q.shape[2]
    plan = pa.MatMulPlan(in_type, out_type, g, m, k, n, options)
    dev = torch.device("cuda:0")

    def buf(which):
        return torch.empty(max(plan.buffer_bytes(which), 1), dtype=torch.uint8,
                           device=dev)

    a, b = device(A_q, in_type), device(B_q, in_type)
    acts, packed, out_int = (buf(capi.BUF_INPUT), buf(capi.BUF_WEIGHTS_PACKED),
                             buf(capi.BUF_OUTPUT))
    ws = buf(capi.BUF_WORKSPACE)
    c = torch.empty((g, m, n), dtype=_TORCH_DTYPE[out_type], device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    plan.pack_rhs(b.data_ptr(), packed.data_ptr(), stream)
    if g == 1:      # the matrices are the convolution's tensors as they stand
        inp, out = a, c
    else:
        plan.lhs_to_internal(a.data_ptr(), acts.data_ptr(), stream)
        inp, out = acts, out_int
    if in_type == pa.QUARTER:
        plan.fwd_quarter(inp.data_ptr(), 0x80, packed.data_ptr(), 0x80,
                         out.data_ptr(), None, ws.data_ptr(),
                         plan.buffer_bytes(capi.BUF_WORKSPACE), stream)
    else:
        plan.fwd(inp.data_ptr(), packed.data_ptr(), out.data_ptr(), None,
                 ws.data_ptr(), plan.buffer_bytes(capi.BUF_WORKSPACE), stream)
    if g != 1:
        plan.out_to_external(out_int.data_ptr(), c.data_ptr(), stream)
    torch.cuda.synchronize()
    result = c.cpu().numpy().astype(np.float64)
    return (result, plan) if return_plan else result


MATMUL_GPU_CASES = [
    # the reference's own harness cases (tests/poplin/CMakeLists.txt:521-880)
    (pa.HALF, pa.HALF, 1, 5, 0, 4, None, None),
    (pa.HALF, pa.HALF, 3, 5, 0, 4, None, None),
    (pa.HALF, pa.HALF, 1, 0, 3, 4, None, None),
    (pa.HALF, pa.HALF, 1, 1, 3, 1, None, None),
    (pa.HALF, pa.FLOAT, 1, 1, 1000, 1, None, None),
    (pa.HALF, pa.HALF, 1, 40, 40, 40, None, None),
    (pa.FLOAT, pa.FLOAT, 1, 40, 40, 40, None, None),
    (pa.HALF, pa.FLOAT, 2, 33, 17, 9, None, None),
    # matrix-core kernel: ragged in every dimension, grouped, both tile widths
    (pa.HALF, pa.HALF, 1, 1024, 512, 512, None, "implicit GEMM"),
    (pa.HALF, pa.FLOAT, 1, 1000, 200, 72, None, "implicit GEMM"),
    (pa.HALF, pa.HALF, 3, 300, 72, 136, None, "implicit GEMM"),
    (pa.HALF, pa.HALF, 1, 130, 1032, 24, None, "implicit GEMM"),
    # the streaming kernel of 1x1 convolutions takes k in 128..512, n = 64
    (pa.HALF, pa.HALF, 1, 4100, 256, 64, None, "pointwise streaming"),
    (pa.HALF, pa.FLOAT, 1, 999, 128, 64, None, "pointwise streaming"),
    (pa.HALF, pa.HALF, 2, 700, 512, 64, None, "pointwise streaming"),
    # forced kernels
    (pa.HALF, pa.HALF, 2, 64, 64, 64,
     {"planConstraints": '{"gfx950": {"kernel": "generic"}}'}, "generic direct"),
    (pa.HALF, pa.HALF, 1, 4100, 256, 64,
     {"planConstraints": '{"gfx950": {"kernel": "igemm"}}'}, "implicit GEMM"),
    # k = n = 1 with groups is a depthwise convolution
    (pa.HALF, pa.HALF, 24, 50, 1, 1, None, None),
    (pa.FLOAT, pa.FLOAT, 1, 300, 130, 70, None, None),
]


@pytest.mark.gpu
@pytest.mark.parametrize("it,ot,g,m,k,n,options,kernel", MATMUL_GPU_CASES)
def test_matmul_on_gpu_matches_numpy(it, ot, g, m, k, n, options, kernel):
    from gpu_helpers import quantize
    rng = np.random.default_rng(g * 1000003 + m * 1009 + k * 31 + n)
    A_q, A = quantize(rng.standard_normal((g, m, k)), it)
    B_q, B = quantize(rng.standard_normal((g, k, n)) / max(k, 1) ** .5, it)
    got, plan = run_matmul(A_q, B_q, it, ot, options, return_plan=True)
    if kernel:
        assert kernel in plan.describe(), plan.describe()
    want = A @ B
    assert got.shape == want.shape
    if want.size:
        # half results round once (<= 2^-11 relative); fp32 accumulation
        tol = 1e-3 if ot == pa.HALF else 1e-5
        assert rel_l2(got, want) <= tol, (rel_l2(got, want), plan.describe())


@pytest.mark.gpu
@pytest.mark.parametrize("g,m,k,n", [(1, 300, 256, 64), (1, 257, 384, 136),
                                     (2, 100, 40, 24), (1, 33, 7, 5)])
def test_matmul_of_signs_is_exact(g, m, k, n):
    # +-1 operands: every product and every partial sum is an integer of
    # magnitude <= k < 2048, exact in fp16 and fp32 in any summation order.
    rng = np.random.default_rng(k)
    A = rng.choice([-1.0, 1.0], size=(g, m, k))
    B = rng.choice([-1.0, 1.0], size=(g, k, n))
    got = run_matmul(A.astype(np.float16), B.astype(np.float16), pa.HALF,
                     pa.HALF)
    np.testing.assert_array_equal(got, A @ B)


@pytest.mark.gpu
def test_matmul_quarter_on_gpu(oracle):
    from gpu_helpers import quantize
    rng = np.random.default_rng(8)
    g, m, k, n = 1, 200, 256, 128
    A_q, A = quantize(rng.standard_normal((g, m, k)), pa.QUARTER, oracle)
    B_q, B = quantize(rng.standard_normal((g, k, n)) / 16, pa.QUARTER, oracle)
    got, plan = run_matmul(A_q, B_q, pa.QUARTER, pa.HALF, return_plan=True)
    assert "implicit GEMM" in plan.describe()
    assert rel_l2(got, A @ B) <= 1e-3


@pytest.mark.gpu
def test_transposed_rhs_is_the_external_weights_layout():
    # B^T [g][n][k] is the convolution's [G][Co][Ci][1] weights: callers that
    # hold the right-hand side transposed pack it with mxconv_pack_weights.
    import torch
    from gpu_helpers import device, quantize
    rng = np.random.default_rng(9)
    g, m, k, n = 2, 150, 72, 40
    A_q, A = quantize(rng.standard_normal((g, m, k)), pa.HALF)
    Bt_q, Bt = quantize(rng.standard_normal((g, n, k)) / 8, pa.HALF)
    plan = pa.MatMulPlan(pa.HALF, pa.FLOAT, g, m, k, n)
    dev = torch.device("cuda:0")
    a, bt = device(A_q, pa.HALF), device(Bt_q, pa.HALF)
    acts = torch.empty_like(a)
    packed = torch.empty(plan.buffer_bytes(capi.BUF_WEIGHTS_PACKED),
                         dtype=torch.uint8, device=dev)
    out_int = torch.empty((m, g, n), dtype=torch.float32, device=dev)
    c = torch.empty((g, m, n), dtype=torch.float32, device=dev)
    plan.pack_weights(bt.data_ptr(), packed.data_ptr())
    plan.lhs_to_internal(a.data_ptr(), acts.data_ptr())
    assert plan.buffer_bytes(capi.BUF_WORKSPACE) == 0
    plan.fwd(acts.data_ptr(), packed.data_ptr(), out_int.data_ptr())
    plan.out_to_external(out_int.data_ptr(), c.data_ptr())
    torch.cuda.synchronize()
    want = A @ Bt.transpose(0, 2, 1)
    assert rel_l2(c.cpu().numpy().astype(np.float64), want) <= 1e-5

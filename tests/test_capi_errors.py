"""Error paths of the C ABI that are decided on the host, before any launch:
short or missing workspaces and buffers, null arguments, unsupported types.
No GPU needed: the pointers given are never dereferenced.  (Reference
counterpart: the shape and argument checks of lib/poplin/Convolution.cpp:105-162
and the option errors of tests/poplin/ConvTest.cpp:684-698.)"""
import ctypes
import json

import pytest

import poplibs_amd as pa
from poplibs_amd import capi
from poplibs_amd.capi import MxconvError, Status
from helpers import make_params

FAKE = 0x1000  # a device "pointer" no checked path touches


def _split_k_plan():
    p = make_params(pa.HALF, batch=4, field=(14, 14), kernel=(3, 3), ci=256,
                    co=256, pad=1)
    # (without the constraint the planner prefers the resident-patch kernel,
    # which needs no workspace)
    plan = pa.Plan(p, {"planConstraints": '{"gfx950": {"patch": 0}}'})
    assert "K split" in plan.describe()
    assert plan.buffer_bytes(capi.BUF_WORKSPACE) > 0
    return plan


def test_fwd_reports_a_short_or_missing_workspace():
    plan = _split_k_plan()
    need = plan.buffer_bytes(capi.BUF_WORKSPACE)
    for ws, nbytes in ((FAKE, need - 1), (None, need), (None, 0)):
        with pytest.raises(MxconvError) as e:
            plan.fwd(FAKE, FAKE, FAKE, None, ws, nbytes)
        assert e.value.status == Status.WORKSPACE_TOO_SMALL
        assert str(need) in str(e.value)


def test_fwd_null_operands():
    plan = _split_k_plan()
    need = plan.buffer_bytes(capi.BUF_WORKSPACE)
    for args in ((None, FAKE, FAKE), (FAKE, None, FAKE), (FAKE, FAKE, None)):
        with pytest.raises(MxconvError) as e:
            plan.fwd(*args, None, FAKE, need)
        assert e.value.status == Status.NULL_ARGUMENT
    assert pa.lib().mxconv_fwd(None, FAKE, FAKE, None, FAKE, None, 0, None) \
        == Status.NULL_ARGUMENT


def test_fwd_wrong_entry_point_for_the_type():
    half = _split_k_plan()
    with pytest.raises(MxconvError) as e:
        half.fwd_quarter(FAKE, 0x80, FAKE, 0x80, FAKE)
    assert e.value.status == Status.INVALID_PARAMS
    q = pa.Plan(make_params(pa.QUARTER, pa.HALF, batch=2, field=(8, 8),
                            kernel=(3, 3), ci=32, co=32, pad=1))
    with pytest.raises(MxconvError) as e:
        q.fwd(FAKE, FAKE, FAKE)
    assert e.value.status == Status.INVALID_PARAMS
    assert "mxconv_fwd_quarter" in str(e.value)


def test_plan_describe_short_buffer():
    plan = _split_k_plan()
    L = pa.lib()
    need = ctypes.c_size_t()
    assert L.mxconv_plan_describe(plan._h, None, 0, ctypes.byref(need)) \
        == Status.OK
    assert need.value > 100
    buf = ctypes.create_string_buffer(16)
    got = ctypes.c_size_t()
    assert L.mxconv_plan_describe(plan._h, buf, 16, ctypes.byref(got)) \
        == Status.BUFFER_TOO_SMALL
    assert got.value == need.value
    assert b"truncated" in L.mxconv_last_error()
    assert len(buf.value) <= 15  # still terminated


def test_plan_queries_refuse_null_arguments():
    """The calls that only read a plan (costs, detailed costs, constraints)
    check their pointers like the launching ones."""
    plan = _split_k_plan()
    L = pa.lib()
    costs = capi.DetailedCosts()
    u64 = ctypes.c_uint64()
    need = ctypes.c_size_t()
    assert L.mxconv_plan_detailed_costs(None, ctypes.byref(costs)) \
        == Status.NULL_ARGUMENT
    assert L.mxconv_plan_detailed_costs(plan._h, None) == Status.NULL_ARGUMENT
    assert L.mxconv_plan_estimated_costs(None, ctypes.byref(u64),
                                         ctypes.byref(u64)) \
        == Status.NULL_ARGUMENT
    assert L.mxconv_plan_estimated_costs(plan._h, None, ctypes.byref(u64)) \
        == Status.NULL_ARGUMENT
    assert L.mxconv_plan_constraints(None, None, 0, ctypes.byref(need)) \
        == Status.NULL_ARGUMENT
    # and a short buffer for the constraints document reports its size
    assert L.mxconv_plan_constraints(plan._h, None, 0, ctypes.byref(need)) \
        == Status.OK
    buf = ctypes.create_string_buffer(8)
    got = ctypes.c_size_t()
    assert L.mxconv_plan_constraints(plan._h, buf, 8, ctypes.byref(got)) \
        == Status.BUFFER_TOO_SMALL
    assert got.value == need.value > 8
    whole = ctypes.create_string_buffer(need.value)
    assert L.mxconv_plan_constraints(plan._h, whole, need.value,
                                     ctypes.byref(got)) == Status.OK
    assert json.loads(whole.value)["gfx950"]["patch"] == 0


def test_weight_update_workspace_and_type_checks():
    fwd = make_params(pa.HALF, batch=8, field=(14, 14), kernel=(3, 3), ci=64,
                      co=64, pad=1)
    plan = pa.WeightUpdatePlan(fwd)
    need = plan.workspace_bytes()
    assert need > 0
    with pytest.raises(MxconvError) as e:
        plan.calculate_weight_deltas(FAKE, FAKE, FAKE, FAKE, need - 1)
    assert e.value.status == Status.WORKSPACE_TOO_SMALL
    with pytest.raises(MxconvError) as e:
        plan.calculate_weight_deltas(FAKE, FAKE, FAKE, None, need)
    assert e.value.status == Status.WORKSPACE_TOO_SMALL
    with pytest.raises(MxconvError) as e:
        plan.calculate_weight_deltas(FAKE, FAKE, None, FAKE, need)
    assert e.value.status == Status.NULL_ARGUMENT
    with pytest.raises(MxconvError) as e:
        plan.weight_update(FAKE, FAKE, FAKE, 0.1, FAKE, need - 1)
    assert e.value.status == Status.WORKSPACE_TOO_SMALL
    # quarter tensors: the pass is not offered
    q = pa.WeightUpdatePlan(make_params(pa.QUARTER, pa.HALF, batch=8,
                                        field=(6, 6), kernel=(3, 3), ci=16,
                                        co=16, pad=1))
    with pytest.raises(MxconvError) as e:
        q.calculate_weight_deltas(FAKE, FAKE, FAKE, FAKE, 1 << 30)
    assert e.value.status == Status.UNSUPPORTED


def test_static_scratch_refuses_a_plan_beyond_its_buffer():
    p = make_params(pa.HALF, batch=16, field=(56, 56), kernel=(3, 3), ci=64,
                    co=64, pad=1)
    opts = {"planConstraints": json.dumps({"gfx950": {"splitK": 9,
                                                      "patch": 0}})}
    plan = pa.Plan(p, opts)
    assert plan.buffer_bytes(capi.BUF_WORKSPACE) > 32 << 20
    with pytest.raises(MxconvError) as e:
        plan.fwd_static_scratch(FAKE, FAKE, FAKE)
    assert e.value.status == Status.WORKSPACE_TOO_SMALL
    assert "built-in buffer" in str(e.value)


def test_plans_pack_alike():
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    a, b = pa.Plan(p), pa.Plan(p)
    assert a.packs_like(b)
    off = {"planConstraints": json.dumps({"gfx950": {"patch": 0}})}
    assert not a.packs_like(pa.Plan(p, off))
    n64 = {"planConstraints": json.dumps({"gfx950": {"patch": 0,
                                                     "blockN": 64}})}
    assert pa.Plan(p, off).packs_like(pa.Plan(p, n64)) == \
        (pa.Plan(p, off).buffer_bytes(capi.BUF_WEIGHTS_PACKED) ==
         pa.Plan(p, n64).buffer_bytes(capi.BUF_WEIGHTS_PACKED))
    generic = {"planConstraints": json.dumps({"gfx950":
                                              {"kernel": "generic"}})}
    assert not a.packs_like(pa.Plan(p, generic))

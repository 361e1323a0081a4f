"""Several convolutions handed to the device together
(poplin::multiconv::convolution, include/poplin/MultiConvolution.hpp:143-149):
each result must be what the single-convolution entry point gives, whether
convolutions share a launch ("parallel") or run in order ("serial")."""
import numpy as np
import pytest

import poplibs_amd as pa
from poplibs_amd import capi
from helpers import make_params, rel_l2


def test_multiconv_options():
    # lib/poplin/ConvPlan.cpp:1929-1953
    assert pa.multiconv_validate_options({}) is True
    assert pa.multiconv_validate_options({"planType": "serial"}) is False
    assert pa.multiconv_validate_options(
        {"planType": "parallel", "perConvReservedTiles": "50",
         "cycleBackOff": "0.1"}) is True
    for bad in ({"planType": "sideways"}, {"perConvReservedTiles": "many"},
                {"perConvReservedTiles": "-1"}, {"cycleBackOff": "slow"},
                {"partialsType": "half"}):
        with pytest.raises(pa.MxconvError) as e:
            pa.multiconv_validate_options(bad)
        assert e.value.status == pa.Status.INVALID_OPTION, bad


def test_multi_fwd_of_nothing_is_ok():
    pa.multi_fwd([], [], [], [])


MULTI_CASES = [
    dict(batch=2, field=(14, 14), kernel=(3, 3), ci=32, co=32, pad=1),
    dict(batch=1, field=(28, 28), kernel=(5, 5), groups=24),
    dict(batch=2, field=(17, 32), kernel=(1, 1), ci=16, co=16),
    dict(batch=3, field=(9, 10), kernel=(3, 3), ci=8, co=16, stride=2, pad=1),
    dict(batch=2, field=(12, 12), kernel=(1, 1), ci=128, co=64),
    dict(batch=0, field=(4, 4), kernel=(3, 3), ci=4, co=4),
    dict(batch=1, field=(7,), kernel=(3,), ci=3, co=5, kdil=2),
    # three more for the matrix cores with the first one's kernel (half in and
    # out, 128-wide tile, whole k-steps per tap), one of them split along K
    # when it runs alone: they share a launch
    dict(batch=1, field=(9, 9), kernel=(1, 1), ci=64, co=136),
    dict(batch=3, field=(5, 6), kernel=(2, 2), ci=128, co=200, stride=2),
    dict(batch=1, field=(6, 6), kernel=(3, 3), ci=512, co=128, pad=1),
    # and two with the narrow tile and per-lane taps
    dict(batch=2, field=(8, 8), kernel=(3, 3), ci=8, co=24, pad=1),
    dict(batch=1, field=(10, 4), kernel=(1, 3), ci=24, co=40),
    # launches with more to them than one kernel - a padded copy of the
    # input, phases of a dilated input, a padded output field - run on their
    # own inside the set
    dict(batch=4, field=(16, 16), kernel=(3, 3), ci=3, co=128, pad=1),
    dict(batch=2, field=(9, 8), kernel=(3, 3), ci=64, co=136, idil=2, pad=2),
    dict(batch=2, field=(9, 8), kernel=(3, 3), ci=64, co=136, pad=1,
         opl=(1, 0), opu=(0, 2)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("parallel", [True, False])
def test_multi_fwd_equals_single_convolutions(oracle, parallel):
    import torch
    from gpu_helpers import _TORCH_DTYPE, device, quantize, run_conv
    rng = np.random.default_rng(41)
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    plans, ins, ws, outs, keep, singles, params = [], [], [], [], [], [], []
    wss, wsb = [], []
    for i, kw in enumerate(MULTI_CASES):
        t = pa.FLOAT if i in (2, 5) else pa.HALF
        p = make_params(t, **kw)
        G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                     p.outputChannelsPerConvGroup)
        xq, _ = quantize(rng.standard_normal(
            (p.batchSize, G * Ci, *p.inputFieldShape)), t)
        wq, _ = quantize(rng.standard_normal(
            (G, Co, Ci, *p.kernelShape)) * 0.1, t)
        plan = pa.Plan(p)
        singles.append(run_conv(p, xq, wq, plan=plan))

        def buf(which):
            return torch.empty(max(plan.buffer_bytes(which), 1),
                               dtype=torch.uint8, device=dev)

        x_ext, w_ext = device(xq, t), device(wq, t)
        x_int, w_pack, o_int = (buf(capi.BUF_INPUT),
                                buf(capi.BUF_WEIGHTS_PACKED),
                                buf(capi.BUF_OUTPUT))
        plan.acts_to_internal(x_ext.data_ptr(), x_int.data_ptr(), stream)
        plan.pack_weights(w_ext.data_ptr(), w_pack.data_ptr(), stream)
        scratch = buf(capi.BUF_WORKSPACE)
        plans.append(plan)
        ins.append(x_int.data_ptr())
        ws.append(w_pack.data_ptr())
        outs.append(o_int.data_ptr())
        wss.append(scratch.data_ptr())
        wsb.append(plan.buffer_bytes(capi.BUF_WORKSPACE))
        keep += [x_ext, w_ext, x_int, w_pack, o_int, scratch]
        params.append((p, o_int, t))
    assert any("K split" in p.describe() for p in plans)
    assert any("input channels padded" in p.describe() for p in plans)
    assert any("phases" in p.describe() for p in plans)
    # twice, with work of the caller's stream in between
    for _ in range(2):
        pa.multi_fwd(plans, ins, ws, outs, workspaces=wss,
                     workspace_bytes=wsb, parallel=parallel, stream=stream)
        torch.cuda.synchronize()
        for (p, o_int, t), plan, want in zip(params, plans, singles):
            o_ext = torch.empty(
                (p.batchSize, p.getNumOutputChans(), *p.getOutputFieldShape()),
                dtype=_TORCH_DTYPE[t], device=dev)
            plan.acts_to_external(o_int.data_ptr(), o_ext.data_ptr(), stream)
            torch.cuda.synchronize()
            got = o_ext.cpu().numpy().astype(np.float64)
            if parallel and "K split" in plan.describe():
                # in a shared launch K stays in one piece: another summation
                # order than the plan's own
                assert rel_l2(got, want) <= 1e-3
            else:
                np.testing.assert_array_equal(got, want)
            o_int.zero_()


@pytest.mark.gpu
def test_shared_launch_with_biases_and_groups(oracle):
    # three convolutions of one kernel instantiation, each with its own bias
    # (one without), one of them grouped: the shared launch takes each
    # member's own arguments
    import torch
    from gpu_helpers import device, quantize, run_conv
    rng = np.random.default_rng(43)
    dev = torch.device("cuda:0")
    cases = [(dict(batch=2, field=(6, 7), kernel=(3, 3), ci=64, co=72, pad=1),
              True),
             (dict(batch=1, field=(9, 9), kernel=(1, 1), ci=128, co=130), False),
             (dict(batch=2, field=(5, 5), kernel=(2, 2), ci=64, co=80,
                   groups=2), True)]
    plans, ins, ws, outs, biases, keep, want, shapes = ([], [], [], [], [], [],
                                                       [], [])
    for kw, with_bias in cases:
        p = make_params(pa.HALF, pa.FLOAT, **kw)
        G, Ci, Co = (p.numConvGroups, p.inputChannelsPerConvGroup,
                     p.outputChannelsPerConvGroup)
        xq, _ = quantize(rng.standard_normal(
            (p.batchSize, G * Ci, *p.inputFieldShape)), pa.HALF)
        wq, _ = quantize(rng.standard_normal(
            (G, Co, Ci, *p.kernelShape)) * 0.1, pa.HALF)
        bq, _ = quantize(rng.standard_normal(G * Co), pa.FLOAT)
        plan = pa.Plan(p)
        assert "K split" not in plan.describe()
        want.append(run_conv(p, xq, wq, bq if with_bias else None, plan=plan))
        x_ext, w_ext = device(xq, pa.HALF), device(wq, pa.HALF)
        x_int = torch.empty(plan.buffer_bytes(capi.BUF_INPUT),
                            dtype=torch.uint8, device=dev)
        w_pack = torch.empty(plan.buffer_bytes(capi.BUF_WEIGHTS_PACKED),
                             dtype=torch.uint8, device=dev)
        o_int = torch.empty(plan.buffer_bytes(capi.BUF_OUTPUT),
                            dtype=torch.uint8, device=dev)
        b_dev = device(bq, pa.FLOAT)
        plan.acts_to_internal(x_ext.data_ptr(), x_int.data_ptr())
        plan.pack_weights(w_ext.data_ptr(), w_pack.data_ptr())
        plans.append(plan)
        ins.append(x_int.data_ptr())
        ws.append(w_pack.data_ptr())
        outs.append(o_int.data_ptr())
        biases.append(b_dev.data_ptr() if with_bias else None)
        keep += [x_ext, w_ext, x_int, w_pack, o_int, b_dev]
        shapes.append((p.batchSize, G * Co, *p.getOutputFieldShape()))
    pa.multi_fwd(plans, ins, ws, outs, biases=biases)
    torch.cuda.synchronize()
    for plan, o_ptr, w, shape in zip(plans, outs, want, shapes):
        o_ext = torch.empty(shape, dtype=torch.float32, device=dev)
        plan.acts_to_external(o_ptr, o_ext.data_ptr())
        torch.cuda.synchronize()
        np.testing.assert_array_equal(o_ext.cpu().numpy().astype(np.float64),
                                      w)


@pytest.mark.gpu
def test_multi_fwd_quarter_metadata(oracle):
    import torch
    from gpu_helpers import device, quantize, run_conv
    rng = np.random.default_rng(42)
    dev = torch.device("cuda:0")
    p = make_params(pa.QUARTER, pa.HALF, batch=2, field=(8, 8), kernel=(3, 3),
                    ci=32, co=16, pad=1)
    metas = [(0x81, 0x02), (0x3f, 0x80)]   # (format, scale) pairs differ
    plans, ins, ws, outs, keep, want = [], [], [], [], [], []
    for in_meta, w_meta in metas:
        xq, _ = quantize(rng.standard_normal((2, 32, 8, 8)), pa.QUARTER, oracle)
        wq, _ = quantize(rng.standard_normal((1, 16, 32, 3, 3)) * 0.2,
                         pa.QUARTER, oracle)
        plan = pa.Plan(p)
        want.append(run_conv(p, xq, wq, plan=plan, in_meta=in_meta,
                             w_meta=w_meta))
        x_ext, w_ext = device(xq, pa.QUARTER), device(wq, pa.QUARTER)
        x_int = torch.empty(plan.buffer_bytes(capi.BUF_INPUT),
                            dtype=torch.uint8, device=dev)
        w_pack = torch.empty(plan.buffer_bytes(capi.BUF_WEIGHTS_PACKED),
                             dtype=torch.uint8, device=dev)
        o_int = torch.empty(plan.buffer_bytes(capi.BUF_OUTPUT),
                            dtype=torch.uint8, device=dev)
        plan.acts_to_internal(x_ext.data_ptr(), x_int.data_ptr())
        plan.pack_weights(w_ext.data_ptr(), w_pack.data_ptr())
        plans.append(plan)
        ins.append(x_int.data_ptr())
        ws.append(w_pack.data_ptr())
        outs.append(o_int.data_ptr())
        keep += [x_ext, w_ext, x_int, w_pack, o_int]
    pa.multi_fwd(plans, ins, ws, outs, in_metadata=[m[0] for m in metas],
                 weights_metadata=[m[1] for m in metas])
    torch.cuda.synchronize()
    for plan, o_ptr, w in zip(plans, outs, want):
        o_ext = torch.empty((2, 16, 8, 8), dtype=torch.float16, device=dev)
        plan.acts_to_external(o_ptr, o_ext.data_ptr())
        torch.cuda.synchronize()
        np.testing.assert_array_equal(o_ext.cpu().numpy().astype(np.float64),
                                      w)

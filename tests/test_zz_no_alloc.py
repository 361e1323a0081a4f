"""The forward entry point that allocates nothing, mxconv_fwd_static_scratch,
against mxconv_fwd on plans that need scratch memory (K split over workgroups;
input channels padded to a whole vector): bit-identical outputs (the same
kernels run), on two calls in a row, the second with a smaller input, and a
clear refusal of a plan whose workspace exceeds the built-in buffer."""
import json

import numpy as np
import pytest
import torch

import poplibs_amd as pa
from poplibs_amd import capi
from helpers import make_params, random_data

pytestmark = pytest.mark.gpu


def _both(p, seed, options=None, setup=False):
    from gpu_helpers import quantize, device
    plan = pa.Plan(p, options)
    need = plan.buffer_bytes(capi.BUF_WORKSPACE)
    assert need > 0, plan.describe()
    acts, weights, biases = random_data(p, seed, "normal")
    aq, _ = quantize(acts, p.inputType)
    wq, _ = quantize(weights * 0.1, p.inputType)
    bq, _ = quantize(biases, p.outputType)
    dev = torch.device("cuda:0")

    def buf(which):
        return torch.empty(max(plan.buffer_bytes(which), 1),
                           dtype=torch.uint8, device=dev)

    a_ext, w_ext = device(aq, p.inputType), device(wq, p.inputType)
    bias = device(bq, p.outputType)
    a_int, w_pack = buf(capi.BUF_INPUT), buf(capi.BUF_WEIGHTS_PACKED)
    ws = buf(capi.BUF_WORKSPACE)
    s = torch.cuda.current_stream().cuda_stream
    plan.acts_to_internal(a_ext.data_ptr(), a_int.data_ptr(), s)
    plan.pack_weights(w_ext.data_ptr(), w_pack.data_ptr(), s)
    want = buf(capi.BUF_OUTPUT).zero_()
    got = buf(capi.BUF_OUTPUT).fill_(0xAB)
    plan.fwd(a_int.data_ptr(), w_pack.data_ptr(), want.data_ptr(),
             bias.data_ptr(), ws.data_ptr(), need, s)
    # (device memory as the driver counts it: an allocation by anybody would
    # show; torch's own counter may only fall - the collector freeing tensors
    # of earlier tests)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    before = torch.cuda.memory_allocated()
    plan.fwd_static_scratch(a_int.data_ptr(), w_pack.data_ptr(),
                            got.data_ptr(), bias.data_ptr(), s)
    torch.cuda.synchronize()
    if not setup:
        assert torch.cuda.memory_allocated() <= before
        assert torch.cuda.mem_get_info()[0] == free_before
    n = plan.buffer_bytes(capi.BUF_OUTPUT)
    np.testing.assert_array_equal(got[:n].cpu().numpy(),
                                  want[:n].cpu().numpy())
    assert want[:n].any()


# The planner prefers the resident-patch kernel for these layers, which needs
# no scratch memory; the streaming kernel with K split is asked for by name.
STREAMING = {"planConstraints": json.dumps({"gfx950": {"patch": 0}})}


def test_static_scratch_matches_fwd_twice_second_smaller():
    # K split over workgroups: 8 tiles, 36 k-steps
    p = make_params(pa.HALF, batch=4, field=(14, 14), kernel=(3, 3), ci=256,
                    co=256, pad=1)
    assert "K split" in pa.Plan(p, STREAMING).describe()
    # (set-up: the first call on a device looks up the built-in buffer, and
    # the runtime loads the library's device data with it)
    _both(p, 30, STREAMING, setup=True)
    _both(p, 31, STREAMING)
    q = make_params(pa.HALF, batch=1, field=(9, 7), kernel=(3, 3), ci=256,
                    co=128, pad=1)
    assert "K split" in pa.Plan(q, STREAMING).describe()
    _both(q, 32, STREAMING)
    # ... and once more the larger one: nothing of the smaller call is left
    _both(p, 33, STREAMING)


def test_static_scratch_padded_channels_float_out():
    # 5 input channels: a zero-filled copy [pixels][8] goes to the scratch
    p = make_params(pa.HALF, pa.FLOAT, batch=2, field=(32, 32), kernel=(7, 7),
                    ci=5, co=64, pad=3, stride=2)
    assert "input channels padded" in pa.Plan(p).describe()
    _both(p, 34, setup=True)  # (first call on the device if run by itself)
    _both(p, 34)
    _both(make_params(pa.HALF, pa.FLOAT, batch=1, field=(32, 28),
                      kernel=(7, 7), ci=5, co=64, pad=3, stride=2), 35)


def test_static_scratch_refuses_what_does_not_fit():
    # split K on request: 16 parts x 50176 pixels x 64 channels x 4 bytes
    p = make_params(pa.HALF, batch=16, field=(56, 56), kernel=(3, 3), ci=64,
                    co=64, pad=1)
    opts = {"planConstraints": json.dumps({"gfx950": {"splitK": 9,
                                                      "patch": 0}})}
    plan = pa.Plan(p, opts)
    assert plan.buffer_bytes(capi.BUF_WORKSPACE) > 32 << 20
    with pytest.raises(Exception) as e:
        plan.fwd_static_scratch(1, 1, 1, None, 0)
    assert "built-in buffer" in str(e.value)

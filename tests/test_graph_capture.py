"""Launches recorded into a HIP graph and replayed: every entry point on the
forward path only enqueues kernels on the caller's stream (no allocation, no
memset, no synchronisation), so a captured launch must give, on every replay
and for whatever the buffers hold by then, what the same call gives eagerly."""
import numpy as np
import pytest

import poplibs_amd as pa
from poplibs_amd import capi
from helpers import make_params

pytestmark = pytest.mark.gpu

CASES = [
    # the plain kernel; K split over workgroups (partials and a second kernel)
    dict(batch=2, field=(14, 14), kernel=(3, 3), ci=64, co=128, pad=1),
    dict(batch=1, field=(6, 6), kernel=(3, 3), ci=512, co=128, pad=1),
    # a padded copy of the input, phases of a dilated input, a padded output
    dict(batch=4, field=(16, 16), kernel=(3, 3), ci=3, co=32, idil=2, pad=2,
         opl=(1, 0), opu=(0, 1)),
    # pointwise and depthwise kernels
    dict(batch=2, field=(12, 12), kernel=(1, 1), ci=128, co=64),
    dict(batch=2, field=(13, 12), kernel=(3, 3), groups=24, stride=2, pad=1),
]


@pytest.mark.parametrize("kw", CASES)
def test_replays_match_eager_launches(kw):
    import torch
    p = make_params(pa.HALF, pa.HALF, **kw)
    plan = pa.Plan(p)
    dev = torch.device("cuda:0")

    def buf(which):
        return torch.zeros(max(plan.buffer_bytes(which), 16),
                           dtype=torch.uint8, device=dev)

    gen = torch.Generator(device=dev).manual_seed(7)
    n_in = plan.buffer_bytes(capi.BUF_INPUT) // 2
    x = torch.zeros(max(n_in, 8), dtype=torch.float16, device=dev)
    w_ext = (torch.randn(max(plan.buffer_bytes(capi.BUF_WEIGHTS_EXTERNAL) // 2,
                             8), generator=gen, device=dev) * 0.1).half()
    bias = torch.randn(p.getNumOutputChans(), generator=gen,
                       device=dev).half()
    w, ws = buf(capi.BUF_WEIGHTS_PACKED), buf(capi.BUF_WORKSPACE)
    out_graph, out_eager = buf(capi.BUF_OUTPUT), buf(capi.BUF_OUTPUT)
    plan.pack_weights(w_ext.data_ptr(), w.data_ptr())
    torch.cuda.synchronize()

    def launch(out, stream):
        plan.fwd(x.data_ptr(), w.data_ptr(), out.data_ptr(), bias.data_ptr(),
                 ws.data_ptr(), ws.numel(), stream)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        launch(out_graph, side.cuda_stream)      # warm-up outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            launch(out_graph, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for replay in range(3):
        # new input values each time, written by ordinary work of the program
        x.copy_(torch.randn(x.shape, generator=gen, device=dev).half())
        out_graph.fill_(0x5a)
        torch.cuda.synchronize()
        graph.replay()
        launch(out_eager, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(out_graph, out_eager), (replay, plan.describe())
        assert np.isfinite(out_eager.view(torch.float16).float().cpu().numpy()
                           ).all()

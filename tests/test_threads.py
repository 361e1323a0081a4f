"""Host threads.  The reference's API is re-entrant on distinct graphs
(tests/sanity/ParallelTest.cpp:14-30); here plans are immutable once created,
errors are reported per thread, and launches only enqueue work on the
caller's stream - so threads may create plans at the same time and launch
through one shared plan on streams of their own."""
import threading

import numpy as np
import pytest

import poplibs_amd as pa
from poplibs_amd import capi
from poplibs_amd.capi import MxconvError
from helpers import make_params

CASES = [
    dict(batch=2, field=(14, 14), kernel=(3, 3), ci=64, co=128, pad=1),
    dict(batch=1, field=(6, 6), kernel=(3, 3), ci=512, co=128, pad=1),
    dict(batch=4, field=(16, 16), kernel=(3, 3), ci=3, co=32, idil=2, pad=2),
    dict(batch=2, field=(13, 12), kernel=(3, 3), groups=24, stride=2, pad=1),
]


def test_plans_and_errors_from_many_threads():
    """Plan creation side by side; each thread sees its own error message."""
    failures = []

    def work(i):
        try:
            for rep in range(20):
                kw = CASES[(i + rep) % len(CASES)]
                good = pa.Plan(make_params(pa.HALF, pa.HALF, **kw))
                assert "kernel" in good.describe()
                with pytest.raises(MxconvError) as e:
                    pa.Plan(make_params(pa.HALF, pa.HALF, **kw),
                            {"noSuchOption%d" % i: "1"})
                assert "noSuchOption%d" % i in str(e.value), str(e.value)
        except BaseException as ex:  # noqa: BLE001 - reported below
            failures.append((i, repr(ex)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures


@pytest.mark.gpu
@pytest.mark.parametrize("kw", CASES)
def test_one_plan_launched_from_several_threads(kw):
    import torch
    p = make_params(pa.HALF, pa.HALF, **kw)
    plan = pa.Plan(p)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(11)

    def buf(which):
        return torch.zeros(max(plan.buffer_bytes(which), 16),
                           dtype=torch.uint8, device=dev)

    w_ext = (torch.randn(max(plan.buffer_bytes(capi.BUF_WEIGHTS_EXTERNAL) // 2,
                             8), generator=gen, device=dev) * 0.1).half()
    w = buf(capi.BUF_WEIGHTS_PACKED)
    plan.pack_weights(w_ext.data_ptr(), w.data_ptr())
    n_threads, n_in = 4, max(plan.buffer_bytes(capi.BUF_INPUT) // 2, 8)
    inputs = [torch.randn(n_in, generator=gen, device=dev).half()
              for _ in range(n_threads)]
    torch.cuda.synchronize()

    def run(i, stream, out, ws):
        plan.fwd(inputs[i].data_ptr(), w.data_ptr(), out.data_ptr(), None,
                 ws.data_ptr(), ws.numel(), stream)

    # one after the other first: what every thread has to reproduce
    want = []
    for i in range(n_threads):
        out, ws = buf(capi.BUF_OUTPUT), buf(capi.BUF_WORKSPACE)
        run(i, torch.cuda.current_stream().cuda_stream, out, ws)
        torch.cuda.synchronize()
        want.append(out.clone())

    got = [None] * n_threads
    failures = []

    def work(i):
        try:
            stream = torch.cuda.Stream()
            out, ws = buf(capi.BUF_OUTPUT), buf(capi.BUF_WORKSPACE)
            torch.cuda.synchronize()
            for _ in range(10):
                out.fill_(0x33)
                stream.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(stream):
                    run(i, stream.cuda_stream, out, ws)
                stream.synchronize()
            got[i] = out
        except BaseException as ex:  # noqa: BLE001 - reported below
            failures.append((i, repr(ex)))

    threads = [threading.Thread(target=work, args=(i,))
               for i in range(n_threads)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not failures, failures
    for i in range(n_threads):
        assert torch.equal(got[i], want[i]), i
    assert np.isfinite(want[0].view(torch.float16).float().cpu().numpy()).all()

#!/usr/bin/env python3
"""Benchmark of the MI355X forward convolution behind the C ABI.

A "step" is one forward convolution (one `mxconv_fwd` call) over one batch of
synthetic, seeded input that is already resident in HBM in the device layout
(channels-last activations, packed weights).  The headline workload is the
ResNet-style 3x3 layer the metric is quoted on; the other configurations
(1x1, depthwise, fp8) are measured the same way and reported inside the same
JSON line under "other_workloads", and the backward-data and weight-delta
passes of the 3x3 and the depthwise layer under "training_passes".

    python bench.py --gpus 1 --steps K --warmup W

prints ONE JSON line.  Only one GPU is used; --gpus above 1 is refused.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"fp16": 2500.0, "fp8": 5000.0}   # MI355X dense MFMA
PEAK_HBM_GBS = 8000.0                            # MI355X HBM3E


def _workloads(pa):
    """The benchmark configurations 2-5 as ConvParams + data recipe."""
    def params(t_in, t_out, batch, field, kernel, ci, co, groups, stride, pad):
        p = pa.ConvParams(t_in, t_out, batch, list(field), list(kernel), ci,
                          co, groups)
        p.inputTransform.paddingLower = [pad] * len(field)
        p.inputTransform.paddingUpper = [pad] * len(field)
        p.outputTransform.stride = [stride] * len(field)
        return p
    return {
        "c2": dict(
            name="configs[1]: ResNet-style 3x3 conv N=32 28x28 Cin=Cout=128 "
                 "stride 1 pad 1, fp16 in/weights, fp32 partials, fp16 out",
            params=params(pa.HALF, pa.HALF, 32, (28, 28), (3, 3), 128, 128, 1,
                          1, 1),
            dtype="fp16", bound="mfma", relu=False, w_std=(2 / (9 * 128)) ** .5),
        "c3": dict(
            name="configs[2]: 1x1 conv N=32 56x56 Cin=256 Cout=64, fp16",
            params=params(pa.HALF, pa.HALF, 32, (56, 56), (1, 1), 256, 64, 1,
                          1, 0),
            dtype="fp16", bound="hbm", relu=True, w_std=(2 / 256) ** .5),
        "c4": dict(
            name="configs[3]: depthwise 3x3 stride 2 pad 1 N=32 112x112 C=96, "
                 "fp16 in, fp32 partials, fp16 out",
            params=params(pa.HALF, pa.HALF, 32, (112, 112), (3, 3), 1, 1, 96,
                          2, 1),
            dtype="fp16", bound="hbm", relu=False, w_std=(2 / 9) ** .5),
        "c5": dict(
            name="configs[4]: fp8 E4M3 3x3 conv N=64 14x14 Cin=Cout=256 "
                 "stride 1 pad 1, per-tensor 2^k scales, fp32 acc, fp16 out",
            params=params(pa.QUARTER, pa.HALF, 64, (14, 14), (3, 3), 256, 256,
                          1, 1, 1),
            dtype="fp8", bound="mfma", relu=False,
            w_std=(2 / (9 * 256)) ** .5),
        # Not one of the benchmark configurations: a layer that fills the chip
        # seven times over, where the launch is a small part of the time.
        "steady_state": dict(
            name="steady state (not a benchmark configuration): 3x3 conv "
                 "N=128 28x28 Cin=Cout=256 stride 1 pad 1, fp16, 1792 tiles "
                 "= 7 rounds on 256 CUs",
            params=params(pa.HALF, pa.HALF, 128, (28, 28), (3, 3), 256, 256,
                          1, 1, 1),
            dtype="fp16", bound="mfma", relu=False,
            w_std=(2 / (9 * 256)) ** .5),
        # ... and a first layer: three input channels, read as they are.
        "first_layer": dict(
            name="first layer (not a benchmark configuration): 7x7 conv "
                 "stride 2 pad 3 N=32 224x224 Cin=3 Cout=64, fp16",
            params=params(pa.HALF, pa.HALF, 32, (224, 224), (7, 7), 3, 64, 1,
                          2, 3),
            dtype="fp16", bound="hbm", relu=False, w_std=(2 / 147) ** .5),
    }


class Runner:
    """Device buffers + plan of one workload; `launch(i)` enqueues one
    forward convolution on buffer set i."""

    def __init__(self, pa, capi, torch, wl, seed=0, sets=1):
        self.pa, self.torch, self.wl = pa, torch, wl
        p = self.p = wl["params"]
        self.plan = pa.Plan(p)
        dev = torch.device("cuda:0")
        from poplibs_amd import synthetic
        ashape = (p.batchSize, p.getNumInputChans(), *p.inputFieldShape)
        wshape = (p.numConvGroups, p.outputChannelsPerConvGroup,
                  p.inputChannelsPerConvGroup, *p.kernelShape)
        # mt19937_64(seed) for the activations, (seed + 1) for the weights,
        # Box-Muller normals, drawn in the order of the external arrays
        acts = torch.from_numpy(synthetic.normal(seed, ashape))
        if wl["relu"]:
            acts = acts.clamp_min(0)
        weights = torch.from_numpy(
            synthetic.normal(seed + 1, wshape, wl["w_std"]))
        self.in_meta = self.w_meta = 0x80
        if p.inputType == pa.QUARTER:
            import math
            sa = math.ceil(math.log2(acts.abs().max().item() / 448.0))
            sw = math.ceil(math.log2(weights.abs().max().item() / 448.0))
            self.in_meta = pa.quarter_metadata(1, sa)
            self.w_meta = pa.quarter_metadata(1, sw)
            a_ext = (acts / 2.0 ** sa).float().to(
                torch.float8_e4m3fn).view(torch.uint8)
            w_ext = (weights / 2.0 ** sw).float().to(
                torch.float8_e4m3fn).view(torch.uint8)
        else:
            a_ext, w_ext = acts.half(), weights.half()
        self.a_ext_host, self.w_ext_host = a_ext, w_ext
        a_ext, w_ext = a_ext.to(dev), w_ext.to(dev)

        def buf(which):
            return torch.empty(max(self.plan.buffer_bytes(which), 16),
                               dtype=torch.uint8, device=dev)

        self.w_pack = buf(capi.BUF_WEIGHTS_PACKED)
        self.ws = buf(capi.BUF_WORKSPACE)
        self.ws_bytes = self.plan.buffer_bytes(capi.BUF_WORKSPACE)
        s = torch.cuda.current_stream().cuda_stream
        self.plan.pack_weights(w_ext.data_ptr(), self.w_pack.data_ptr(), s)
        self.inputs, self.outputs = [], []
        for _ in range(sets):
            a_int = buf(capi.BUF_INPUT)
            self.plan.acts_to_internal(a_ext.data_ptr(), a_int.data_ptr(), s)
            self.inputs.append(a_int)
            self.outputs.append(buf(capi.BUF_OUTPUT))
        torch.cuda.synchronize()
        self.flops = p.getFwdFlops()
        self.bytes = (self.plan.buffer_bytes(capi.BUF_INPUT)
                      + self.plan.buffer_bytes(capi.BUF_WEIGHTS_EXTERNAL)
                      + self.plan.buffer_bytes(capi.BUF_OUTPUT))

    def launch(self, i=0):
        s = self.torch.cuda.current_stream().cuda_stream
        k = i % len(self.inputs)
        if self.p.inputType == self.pa.QUARTER:
            self.plan.fwd_quarter(self.inputs[k].data_ptr(), self.in_meta,
                                  self.w_pack.data_ptr(), self.w_meta,
                                  self.outputs[k].data_ptr(), None,
                                  self.ws.data_ptr(), self.ws_bytes, s)
        else:
            self.plan.fwd(self.inputs[k].data_ptr(), self.w_pack.data_ptr(),
                          self.outputs[k].data_ptr(), None, self.ws.data_ptr(),
                          self.ws_bytes, s)

    def output_external(self, k=0):
        """Output of buffer set k in the external [B][C][H][W] layout."""
        torch, p = self.torch, self.p
        dt = torch.float16 if p.outputType == self.pa.HALF else torch.float32
        o_ext = torch.empty((p.batchSize, p.getNumOutputChans(),
                             *p.getOutputFieldShape()), dtype=dt,
                            device="cuda:0")
        self.plan.acts_to_external(self.outputs[k].data_ptr(),
                                   o_ext.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return o_ext.cpu().numpy().astype(np.float64)

    def oracle_inputs(self, images):
        """The rounded inputs as float64, for the oracle."""
        import oracle
        a, w = self.a_ext_host[images], self.w_ext_host
        if self.p.inputType == self.pa.QUARTER:
            return (oracle.quarter_to_double(a.numpy(), self.in_meta),
                    oracle.quarter_to_double(w.numpy(), self.w_meta))
        return a.double().numpy(), w.double().numpy()


def time_steps(torch, runner, steps, warmup):
    """Returns (wall seconds for `steps` steps, mean kernel seconds per launch
    from HIP events on the launch stream, how the steps were issued)."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(warmup):
            runner.launch(i)
        stream.synchronize()
        # The steps are recorded once into a HIP graph and replayed, so that
        # what is timed is the GPU work and not the Python launch loop.
        mode = "hipGraph replay of the recorded steps"
        graph = torch.cuda.CUDAGraph()
        try:
            with torch.cuda.graph(graph, stream=stream):
                for i in range(steps):
                    runner.launch(warmup + i)
            graph.replay()  # untimed: instantiation + first upload
            stream.synchronize()
        except Exception as e:  # capture unsupported: eager launches
            graph = None
            mode = f"eager launches (graph capture failed: {e})"
        # A pass = the K steps replayed as often as it takes to fill about
        # 5 ms of GPU time, whatever K is; 7 passes; the median pass is
        # reported (the fastest one beside it).
        def one_pass(replays):
            start = torch.cuda.Event(enable_timing=True)
            stop = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            start.record(stream)
            for _ in range(replays):
                if graph is not None:
                    graph.replay()
                else:
                    for i in range(steps):
                        runner.launch(warmup + i)
            stop.record(stream)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0,
                    start.elapsed_time(stop) * 1e-3)
        _, probe = one_pass(1)
        replays = int(max(1, min(1000, -(-5e-3 // max(probe, 1e-6)))))
        passes = sorted((one_pass(replays) for _ in range(7)),
                        key=lambda x: x[1])
        wall, kernel = passes[len(passes) // 2]
        wall, kernel = wall / replays, kernel / (replays * steps)
        fastest = passes[0][1] / (replays * steps)
        mode += (f", median of 7 timed passes of {replays} x K steps "
                 "(>= 5 ms of GPU time per pass)")
    return wall, kernel, mode, fastest


class TrainingRunner:
    """The backward-data or the weight-delta pass of a workload's layer on
    synthetic tensors resident in HBM; `launch(i)` enqueues one pass."""

    def __init__(self, pa, capi, torch, wl, which):
        self.pa, self.torch = pa, torch
        p = wl["params"]
        dev = torch.device("cuda:0")
        g = torch.Generator(device="cpu").manual_seed(1)

        def randn_half(nbytes):
            return torch.randn(max(nbytes // 2, 8), generator=g,
                               dtype=torch.float32).half().to(dev)

        def buf(nbytes):
            return torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)

        self.flops = p.getFwdFlops()
        in_bytes = pa.Plan(p).buffer_bytes(capi.BUF_INPUT)
        out_bytes = pa.Plan(p).buffer_bytes(capi.BUF_OUTPUT)
        w_bytes = pa.Plan(p).buffer_bytes(capi.BUF_WEIGHTS_EXTERNAL)
        self.bytes = in_bytes + out_bytes + w_bytes
        self.deltas = randn_half(out_bytes)
        if which == "bwd":
            self.plan = pa.Plan(pa.getGradientParams(p))
            self.w_pack = randn_half(
                self.plan.buffer_bytes(capi.BUF_WEIGHTS_PACKED))
            self.result = buf(self.plan.buffer_bytes(capi.BUF_OUTPUT))
            self.ws_bytes = self.plan.buffer_bytes(capi.BUF_WORKSPACE)
            self.ws = buf(self.ws_bytes)
            self.launch = self._bwd
        else:
            self.plan = pa.WeightUpdatePlan(p)
            self.acts = randn_half(in_bytes)
            self.result = buf(w_bytes)
            self.ws_bytes = self.plan.workspace_bytes()
            self.ws = buf(self.ws_bytes)
            self.launch = self._wu
        text = self.plan.describe()
        self.kernel = [l.split("kernel", 1)[1].strip()
                       for l in text.splitlines()
                       if l.strip().startswith("kernel ")][0]
        if which == "wu" and "depthwise weight-delta kernel" in text:
            self.kernel = "depthwise weight-delta kernel (vector ALU)"
            if "streamed through LDS rings" in text:
                self.kernel = ("depthwise weight-delta kernel (vector ALU, "
                               "rows of both tensors streamed through LDS "
                               "rings by persistent workgroups) + ordered sum")
        if which == "wu" and "matrix-core weight-delta kernel" in text:
            self.kernel = ("matrix-core weight-delta kernel on the layer's own "
                           "tensors (MFMA, transposing LDS reads) + ordered sum")

    def _bwd(self, i=0):
        s = self.torch.cuda.current_stream().cuda_stream
        self.plan.fwd(self.deltas.data_ptr(), self.w_pack.data_ptr(),
                      self.result.data_ptr(), None, self.ws.data_ptr(),
                      self.ws_bytes, s)

    def _wu(self, i=0):
        s = self.torch.cuda.current_stream().cuda_stream
        self.plan.calculate_weight_deltas(
            self.deltas.data_ptr(), self.acts.data_ptr(),
            self.result.data_ptr(), self.ws.data_ptr(), self.ws_bytes, s)


def cpu_baseline(runner, tol, budget_s=12.0):
    """Times the single-threaded CPU oracle (a port of the reference's
    poplibs_test::conv::convolution) on a bounded sample of the same
    workload: the first n images of the batch.  The sample's result also
    checks the GPU's output for those images; this is the only place where
    this program runs the oracle."""
    import oracle
    p = runner.p
    one = runner.pa.ConvParams.from_c(p.to_c())
    one.batchSize = 1
    acts, weights = runner.oracle_inputs([0])
    t0 = time.perf_counter()
    oracle.convolution(one, acts, weights, threads=1)
    t1 = time.perf_counter() - t0
    n = int(max(1, min(p.batchSize, round(budget_s / max(t1, 1e-3)))))
    sample = runner.pa.ConvParams.from_c(p.to_c())
    sample.batchSize = n
    acts, weights = runner.oracle_inputs(list(range(n)))
    # A workload the oracle finishes early is repeated, so that the figure
    # rests on about budget_s of CPU work either way.
    reps = int(min(16, max(1, round(budget_s / max(t1 * n, 1e-3))))) \
        if n == p.batchSize else 1
    t0 = time.perf_counter()
    for _ in range(reps):
        want = oracle.convolution(sample, acts, weights, threads=1)
    t = (time.perf_counter() - t0) / reps
    runner.launch(0)
    got = runner.output_external(0)[:n]
    err = float(np.linalg.norm((got - want).ravel())
                / np.linalg.norm(want.ravel()))
    if not err <= tol:
        raise SystemExit(f"parity check failed: rel-L2 {err} > {tol}")
    return {"value": round(sample.getFwdFlops() / t / 1e12, 6),
            "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"first {n} of {p.batchSize} images of the same "
                      f"workload, {reps} x {t:.2f} s, double precision, 1 thread",
            "gpu_rel_l2_vs_sample": err, "tolerance": tol}


def kernel_sources_hash():
    """SHA-256 over the kernel sources (poplibs_amd/csrc), file by file in
    name order: what a counter measurement is stamped with."""
    import hashlib
    h = hashlib.sha256()
    d = os.path.join(ROOT, "poplibs_amd", "csrc")
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".hpp", ".cpp")):
            h.update(name.encode())
            with open(os.path.join(d, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def measured_traffic(key):
    """(HBM bytes per launch from the committed rocprofv3 counter runs or
    None, whether that measurement was taken on other kernel sources than
    the ones in the tree)."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            data = json.load(f)
    except (OSError, ValueError):
        return None, None
    entry = data.get(key, {})
    if "bytes_per_launch" not in entry:
        return None, None
    # (one stamp for the file: all its entries come from one pass)
    stamp = entry.get("kernel_sources_sha256",
                      data.get("kernel_sources_sha256"))
    return entry["bytes_per_launch"], stamp != kernel_sources_hash()


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_reference_c1(pa):
    """configs[0]: the reference's own CPU-runnable case (N=1, 32x32, 16 ->
    16, 3x3, stride 1, pad 1, fp32, uniform[-1, 1) from seed 0), timed on
    the single-threaded oracle: best of 5 runs of a second or so each."""
    import oracle
    from poplibs_amd import synthetic
    p = pa.ConvParams(pa.FLOAT, pa.FLOAT, 1, [32, 32], [3, 3], 16, 16, 1)
    p.inputTransform.paddingLower = [1, 1]
    p.inputTransform.paddingUpper = [1, 1]
    acts = synthetic.uniform(0, (1, 16, 32, 32), -1.0, 1.0).astype(
        np.float32).astype(np.float64)
    weights = synthetic.uniform(1, (1, 16, 16, 3, 3), -1.0, 1.0).astype(
        np.float32).astype(np.float64)
    oracle.convolution(p, acts, weights, threads=1)
    best = float("inf")
    for _ in range(5):
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < 1.0:
            oracle.convolution(p, acts, weights, threads=1)
            n += 1
        best = min(best, (time.perf_counter() - t0) / n)
    return {"workload": "configs[0]: N=1 32x32 16->16 3x3 s1 p1 fp32, "
                        "uniform[-1,1) seed 0",
            "ms": round(best * 1e3, 4),
            "value": round(p.getFwdFlops() / best / 1e9, 4),
            "unit": "GFLOP/s", "flops": p.getFwdFlops(), "cores": 1,
            "kind": "port",
            "sample": "whole workload, best of 5 x ~1 s of repeats, double "
                      "precision, 1 thread"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2",
                    help="headline workload (c2, c3, c4, c5; steady_state)")
    ap.add_argument("--only", action="store_true",
                    help="skip the other workloads and the CPU baseline")
    ap.add_argument("--cache-hot", action="store_true",
                    help="with --only: also time the HBM-bound workload on "
                         "one buffer set (tensors in the Infinity Cache); "
                         "left out by default there, so that a kernel trace "
                         "of the command averages launches of one kind")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 64 MiB device copy, so that a "
                         "counter run of this command holds a kernel of known "
                         "HBM traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no "
                         "multi-GPU path, run with --gpus 1")
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU; there is no CPU fallback")
    import poplibs_amd as pa
    from poplibs_amd import capi
    pa.lib()
    wls = _workloads(pa)
    if args.copy_calibration:
        src = torch.empty(64 * 2 ** 20, dtype=torch.uint8,
                          device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    def measure(key, steps, warmup):
        wl = wls[key]
        # HBM-bound workloads rotate over enough buffer sets to exceed the
        # 256 MB Infinity Cache, so that reads really come from HBM.
        probe = Runner(pa, capi, torch, wl, sets=1)
        sets = 1
        if wl["bound"] == "hbm":
            sets = max(1, -(-300 * 2 ** 20 // probe.bytes))
        runner = probe if sets == 1 else Runner(pa, capi, torch, wl, sets=sets)
        wall, kernel, mode, fastest = time_steps(torch, runner, steps,
                                                 warmup)
        # ... and, labelled as such, the figure with one buffer set (tensors
        # in the Infinity Cache from the launch before)
        hot = None
        if sets != 1 and (args.cache_hot or not args.only):
            _, hot, _, _ = time_steps(torch, probe, steps, warmup)
        if wl["bound"] == "mfma":
            achieved = runner.flops / kernel / 1e12
            peak, unit = PEAK_TFLOPS[wl["dtype"]], "TFLOP/s"
        else:
            achieved = runner.bytes / kernel / 1e9
            peak, unit = PEAK_HBM_GBS, "GB/s"
        traffic, stale = measured_traffic(key)
        return dict(
            runner=runner, wall=wall, kernel=kernel, mode=mode,
            sets=sets,
            roofline={"bound": wl["bound"], "achieved": round(achieved, 3),
                      "peak": peak, "unit": unit,
                      "frac": round(achieved / peak, 4),
                      "traffic": traffic, "traffic_stale": stale,
                      "kernel_us": round(kernel * 1e6, 3),
                      "kernel_us_fastest_pass": round(fastest * 1e6, 3),
                      **({"kernel_us_one_buffer_set_cache_hot":
                          round(hot * 1e6, 3)} if hot else {}),
                      "algorithmic_per_launch":
                          runner.flops if wl["bound"] == "mfma"
                          else runner.bytes})

    head = measure(args.workload, args.steps, args.warmup)
    wl, runner = wls[args.workload], head["runner"]
    tflops = runner.flops * args.steps / head["wall"] / 1e12
    line = {
        "metric": "conv fwd TFLOP/s + % MFMA peak (fp16 3x3 N=32 28x28 "
                  "C=128); depthwise GB/s",
        "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["wall"] * 1e3 / args.steps, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wl["dtype"], "data": "synthetic",
        "config": {"workload": wl["name"], "flops_per_step": runner.flops,
                   "bytes_per_step": runner.bytes,
                   "issue": head["mode"], "buffer_sets": head["sets"],
                   "residency": "HBM-bound workloads rotate over buffer sets "
                                "beyond the 256 MB Infinity Cache; MFMA-bound "
                                "ones reuse one set (operands cache-warm)",
                   "inputs": "mt19937_64(seed 0 / 1), Box-Muller normals, "
                             "rounded to the input type"},
        "roofline": head["roofline"],
    }
    if not args.only:
        others = {}
        for key in wls:
            if key == args.workload:
                continue
            m = measure(key, args.steps, args.warmup)
            r = m["runner"]
            others[key] = {
                "workload": wls[key]["name"],
                "ms_per_step": round(m["wall"] * 1e3 / args.steps, 6),
                "tflops": round(r.flops * args.steps / m["wall"] / 1e12, 3),
                "gbytes_per_s": round(r.bytes * args.steps / m["wall"] / 1e9,
                                      1),
                "buffer_sets": m["sets"],
                "roofline": m["roofline"]}
            del m, r
            torch.cuda.empty_cache()
        line["other_workloads"] = others
        # The layer's other two passes (the rows this build widened into):
        # time per pass, tensors resident in HBM, one buffer set.  Their
        # parity against the oracle is the GPU tests' business.
        passes = {}
        for key in ("c2", "c4"):
            passes[key] = {}
            for which in ("bwd", "wu"):
                r = TrainingRunner(pa, capi, torch, wls[key], which)
                wall, kernel, _, _ = time_steps(torch, r, args.steps,
                                                args.warmup)
                passes[key][which] = {
                    "us_per_pass": round(kernel * 1e6, 2),
                    "tflops": round(r.flops / kernel / 1e12, 2),
                    "gbytes_per_s": round(r.bytes / kernel / 1e9, 1),
                    "kernel": r.kernel}
                del r
                torch.cuda.empty_cache()
        line["training_passes"] = passes
        line["cpu_baseline"] = cpu_baseline(
            runner, 3e-2 if wl["dtype"] == "fp8" else 1e-3)
        line["cpu_baseline"]["cpu_model"] = cpu_model()
        line["cpu_baseline"]["host_cores"] = os.cpu_count()
        line["cpu_baseline"]["configs0"] = cpu_reference_c1(pa)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()

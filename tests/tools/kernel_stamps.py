#!/usr/bin/env python3
"""Per-phase stamps of the benchmark kernels: cycle stamps of
igemmPatch16Kernel (c2, c5), wall-clock milestones of depthwiseRowsKernel (c4).

    python3 tests/tools/kernel_stamps.py [c2|c5] [batch]
    python3 tests/tools/kernel_stamps.py c4

Loads poplibs_amd/libmxconv_stamps.so (the library with the kernel compiled
under -DMXK_PATCH_STAMPS; `make -C poplibs_amd stamps` builds it), runs the
workload the way bench.py does - a HIP graph of 200 launches replayed until
the chip has settled - and prints, for the older (wave 0) and the younger
(wave 4) wave of SIMD 0 of every workgroup of the LAST launch, the mean
number of shader cycles between the kernel's phase boundaries, the shader
clock the chip held (stamp cycles over wall-clock time) and the span from the
first wave's start to the last wave's end.  Diagnostic tool: the stamps cost
the kernel a few hundred cycles, so its total is a little above the product
kernel's.  With a batch size (a multiple of the workload's), the layer is
run at that batch and the table is printed twice: for the workgroups that
start with the launch and for those that start later, on a CU whose
instruction cache an earlier workgroup has filled.

For c4 the table gives, per milestone of the depthwise row-ring kernel, the
time since the first wave of the launch started: mean, earliest and latest
over the 256 workgroups of the last launch of a graph that rotates over four
buffer sets, as bench.py does for the workloads HBM bounds.
"""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

PHASES = [
    (0, 1, "kernel arguments, tile -> pixels -> patch rows, descriptors"),
    (1, 2, "first channel slice of the patch requested"),
    (2, 3, "first k-step's weights requested, pixel offsets"),
    (3, 4, "wait for own part of the slice"),
    (4, 5, "barrier: everybody's part has landed"),
    (5, 6, "other slices and weights requested, first operands read"),
    (6, 7, "k loop (own k-steps)"),
    (7, 8, "K halves handed over through LDS, barrier"),
    (8, 9, "sum, scale / bias, tile to LDS, barrier"),
    (9, 10, "stores issued"),
    (10, 11, "until the last store has landed"),
]


def rows_timeline():
    import torch
    import poplibs_amd.capi as capi
    path = os.path.join(ROOT, "poplibs_amd", "libmxconv_stamps.so")
    if not os.path.exists(path):
        raise SystemExit(f"{path} is missing: make -C poplibs_amd stamps")
    capi._LIB_PATH = path
    import poplibs_amd as pa
    import bench
    lib = pa.lib()
    wl = bench._workloads(pa)["c4"]
    runner = bench.Runner(pa, capi, torch, wl, sets=4)
    text = runner.plan.describe()
    if "LDS ring" not in text:
        raise SystemExit("the plan does not run depthwiseRowsKernel:\n" + text)
    import re
    groups = int(re.search(r"workgroups\s+(\d+) on", text).group(1))
    sink = torch.zeros(groups * 2 * 8, dtype=torch.int64, device="cuda:0")
    lib.mxk_rows_stamp_sink.argtypes = [ctypes.c_void_p]
    lib.mxk_rows_stamp_sink.restype = ctypes.c_int
    if lib.mxk_rows_stamp_sink(sink.data_ptr()) != 0:
        raise SystemExit("mxk_rows_stamp_sink failed")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(20):
            runner.launch(i)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(200):
                runner.launch(i)
        graph.replay()
        stream.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(5):
            graph.replay()
        stop.record(stream)
        stream.synchronize()
    per_launch = start.elapsed_time(stop) * 1e3 / 1000
    d = sink.cpu().numpy().reshape(groups, 2, 8).astype(np.float64) * 10.0
    lib.mxk_rows_stamp_sink(None)
    t0 = d[:, :, 0].min()
    c, l = d[:, 0, :] - t0, d[:, 1, :] - t0
    print(f"workload c4: {wl['name']}")
    print(f"{groups} workgroups; {per_launch:.2f} us per launch (stamped "
          "build, graph replay of 200 launches x 5, four buffer sets)")
    print()
    print("| milestone (ns after the launch's first wave started) | mean | "
          "earliest workgroup | latest |")
    print("|---|---|---|---|")
    rows = [("first loader wave starts", l[:, 0]),
            ("loader: set-up done, first load goes out", l[:, 1]),
            ("loader: the three rows of output row 0 requested", l[:, 2]),
            ("loader: the seven rows of the first three steps requested",
             l[:, 3]),
            ("compute: output row 0's input has landed", c[:, 1]),
            ("compute: output row 1's", c[:, 2]),
            ("compute: the last output row's", c[:, 3]),
            ("loader: last loads landed", l[:, 5]),
            ("compute: last store issued", c[:, 4]),
            ("compute: last store landed", c[:, 5])]
    for name, v in rows:
        print(f"| {name} | {v.mean():.0f} | {v.min():.0f} | {v.max():.0f} |")
    print()
    steps = 12
    rate = (c[:, 3] - c[:, 2]) / steps
    print(f"steady state: {rate.mean():.0f} ns per output row and workgroup "
          f"(fastest workgroup {rate.min():.0f}, slowest {rate.max():.0f}); "
          f"the workgroups' last stores land {c[:, 5].std():.0f} ns (one "
          f"standard deviation) around their mean, and the launch ends with "
          f"the latest, {c[:, 5].max() - c[:, 5].mean():.0f} ns behind the "
          "mean")
    xcd = np.arange(groups) & 7
    print("mean finish by XCD (workgroup number mod 8): " + ", ".join(
        f"{x}: {c[xcd == x, 5].mean():.0f}" for x in range(8)))


def main():
    workload = sys.argv[1] if len(sys.argv) > 1 else "c2"
    if workload == "c4":
        return rows_timeline()
    import torch
    import poplibs_amd.capi as capi
    path = os.path.join(ROOT, "poplibs_amd", "libmxconv_stamps.so")
    if not os.path.exists(path):
        raise SystemExit(f"{path} is missing: make -C poplibs_amd stamps")
    capi._LIB_PATH = path
    import poplibs_amd as pa
    import bench
    lib = pa.lib()
    wl = bench._workloads(pa)[workload]
    if len(sys.argv) > 2:
        wl["params"].batchSize = int(sys.argv[2])
        wl["name"] += f" (batch {sys.argv[2]})"
    runner = bench.Runner(pa, capi, torch, wl)
    text = runner.plan.describe()
    if "16-pixel" not in text and "MFMA blocks of 16" not in text:
        raise SystemExit("the plan does not run igemmPatch16Kernel:\n" + text)
    groups = int(text.split("workgroups")[1].split()[0])
    sink = torch.zeros(groups * 2 * 16, dtype=torch.int64, device="cuda:0")
    lib.mxk_patch_stamp_sink.argtypes = [ctypes.c_void_p]
    lib.mxk_patch_stamp_sink.restype = ctypes.c_int
    if lib.mxk_patch_stamp_sink(sink.data_ptr()) != 0:
        raise SystemExit("mxk_patch_stamp_sink failed")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(20):
            runner.launch(i)
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for i in range(200):
                runner.launch(i)
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        graph.replay()
        stream.synchronize()
        start.record(stream)
        for _ in range(10):
            graph.replay()
        stop.record(stream)
        stream.synchronize()
    per_launch = start.elapsed_time(stop) * 1e3 / 2000
    d = sink.cpu().numpy().reshape(groups, 2, 16).astype(np.float64)
    lib.mxk_patch_stamp_sink(None)
    print(f"workload {workload}: {wl['name']}")
    print(f"{groups} workgroups; {per_launch:.2f} us per launch (stamped "
          "build, graph replay of 200 launches x 10)")
    print()
    def table(d, title):
        print(title)
        print("| phase | wave 0 (older of its SIMD), cycles | wave 4 "
              "(younger), cycles |")
        print("|---|---|---|")
        for a, b, name in PHASES:
            dt = d[:, :, b] - d[:, :, a]
            print(f"| {name} | {dt[:, 0].mean():.0f} | {dt[:, 1].mean():.0f} |")
        total = d[:, :, 11] - d[:, :, 0]
        print(f"| whole wave, first stamp to last | {total[:, 0].mean():.0f} "
              f"| {total[:, 1].mean():.0f} |")
        print()

    if len(sys.argv) > 2:
        t0 = d[:, 0, 14]
        early = t0 < t0.min() + 100  # within a microsecond of the first
        table(d[early], f"{early.sum()} workgroups that start with the launch")
        table(d[~early], f"{(~early).sum()} workgroups that start later")
    table(d, "all workgroups")
    total = d[:, :, 11] - d[:, :, 0]
    first = d[:, :, 6] - d[:, :, 0]
    print(f"cycles before the k loop begins: wave 0 {first[:, 0].mean():.0f}, "
          f"wave 4 {first[:, 1].mean():.0f}; behind its end: wave 0 "
          f"{(d[:, 0, 11] - d[:, 0, 7]).mean():.0f}, wave 4 "
          f"{(d[:, 1, 11] - d[:, 1, 7]).mean():.0f}")
    print("own k-steps per wave:", sorted(set(d[:, :, 12].ravel().astype(int))))
    wall = (d[:, :, 15] - d[:, :, 14]) * 10.0  # s_memrealtime ticks at 100 MHz
    mhz = total / wall * 1e3
    print(f"shader clock (stamp cycles / wall clock): {mhz.mean():.0f} MHz "
          f"(min {mhz.min():.0f}, max {mhz.max():.0f}); a wave lives "
          f"{wall.mean() / 1e3:.2f} us")
    span = (d[:, :, 15].max() - d[:, :, 14].min()) * 10.0
    skew = (d[:, :, 14].max() - d[:, :, 14].min()) * 10.0
    print(f"first wave's start to last wave's end: {span / 1e3:.2f} us; the "
          f"workgroups start within {skew / 1e3:.2f} us of each other")
    mfma = {"c2": 8064, "c5": 8064}.get(workload)
    if mfma:
        loop = (d[:, :, 7] - d[:, :, 6]).max(axis=1).mean()
        print(f"MFMA time of the tile: {mfma} cycles per SIMD = "
              f"{100 * mfma / loop:.0f} % of the longer wave's k loop, "
              f"{100 * mfma / total.max(axis=1).mean():.0f} % of the wave's life")


if __name__ == "__main__":
    main()

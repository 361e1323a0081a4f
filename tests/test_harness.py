"""The single_conv_layer harness: option handling without a GPU, and on the
GPU the cases the reference drives through its own tool
(tests/poplin/CMakeLists.txt:991-3500), each compared with the host model by
the tool itself (exit code 0 = match)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "tests", "tools", "single_conv_layer")


def run(*args, timeout=120):
    if not os.path.exists(TOOL):
        subprocess.check_call(["make", "-C", os.path.dirname(TOOL)],
                              stdout=subprocess.DEVNULL)
    return subprocess.run([TOOL, *args], capture_output=True, text=True,
                          timeout=timeout)


def test_plan_only_reports_flops_and_plan():
    r = run("--input-channels", "128", "--output-channels", "128", "--field",
            "{28,28}", "--kernel-size", "3", "--padding", "1", "--batch-size",
            "32", "--data-type", "half", "--plan-only")
    assert r.returncode == 0, r.stderr
    assert "Forward FLOPs: 7050625024" in r.stdout
    # 3x3 stride 1 "same": going backwards is the same convolution shape
    assert "Backward FLOPs: 7050625024" in r.stdout
    assert "Backward plan:" in r.stdout
    assert "WU FLOPs: 7050625024" in r.stdout
    assert "WU plan:" in r.stdout
    # weight update: batch and input channels exchanged, 28x28 "kernel"
    assert "kernelShape                {28,28}" in r.stdout
    assert "implicit GEMM" in r.stdout
    assert "inputPaddingLower          {1,1}" in r.stdout


def test_plan_only_preplans_and_reports_estimated_costs():
    """The tool plans its passes ahead of use (tools/single_conv_layer.cpp:
    415-417, 831-850) and, with --report-plan, prints each pass's estimated
    cost; --preplan 0 gives the same plans."""
    args = ["--input-channels", "128", "--output-channels", "128", "--field",
            "{28,28}", "--kernel-size", "3", "--padding", "1", "--batch-size",
            "32", "--data-type", "half", "--plan-only"]
    r = run(*args)
    assert r.returncode == 0, r.stderr
    import re
    costs = re.findall(r"estimated cycles: (\d+), temporary memory: (\d+) "
                       r"bytes", r.stdout)
    assert len(costs) == 2, r.stdout  # forward and backward
    for cycles, memory in costs:
        # 8.5 us measured; 2.1 GHz
        assert 8.5 * 0.75 < int(cycles) / 2100 < 8.5 * 1.25
        assert int(memory) == 0
    assert run(*args, "--preplan", "0").stdout == r.stdout


def test_preplan_and_estimated_costs_host_checks():
    """poplin::preplan fills the cache with the plans planning alone makes,
    once per distinct key, or with nothing when an entry is invalid;
    reportPlanEstimatedCosts is within a quarter of the measured times of the
    benchmark configurations (tests/tools/preplan_test.cpp)."""
    tool = os.path.join(ROOT, "tests", "tools", "preplan_test")
    if not os.path.exists(tool):
        subprocess.check_call(["make", "-C", os.path.dirname(tool)],
                              stdout=subprocess.DEVNULL)
    r = subprocess.run([tool], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout


@pytest.mark.gpu
def test_fully_connected_weight_transpose_on_the_device():
    """poplin::fullyConnectedWeightTranspose (include/poplin/Convolution.hpp:
    695-711): the forward weights with the channel axes exchanged and nothing
    flipped, packed for the backward pass's plan - read back through
    readTensor and compared element by element with the exchange done on the
    host, for kernels of one and three taps, two groups, half and float; the
    result is accepted by convolution() of the backward parameters."""
    tool = os.path.join(ROOT, "tests", "tools", "preplan_test")
    r = subprocess.run([tool, "--device"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "device checks passed" in r.stdout


def test_plan_constraints_and_options_are_validated():
    base = ["--input-channels", "16", "--output-channels", "16", "--field",
            "{8,8}", "--kernel-size", "3", "--plan-only"]
    r = run(*base, "--fwd-plan-constraints", '{"method": {"type": "HMAC"}}')
    assert r.returncode == 0 and "generic direct" in r.stdout
    r = run(*base, "--fwd-plan-constraints", '{"method": {"type": "NOPE"}}')
    assert r.returncode == 1 and "Not a valid method type" in r.stderr
    r = run(*base, "--convolution-options", '{"partialsType": "half"}')
    assert r.returncode == 0
    r = run(*base, "--convolution-options", '{"partialsType": "double"}')
    assert r.returncode == 1


def test_usage_errors_exit_1():
    assert run("--input-channels", "1").returncode == 1
    assert run("--input-channels", "1", "--output-channels", "1", "--field",
               "{4}", "--kernel-size", "9", "--plan-only").returncode == 1
    assert run("--bogus").returncode == 1
    assert run("--input-channels", "1", "--output-channels", "1", "--field",
               "{4}", "--kernel-size", "1", "--single-phase",
               "sideways").returncode == 1


# name, arguments: modelled on the reference's ctest entries
GPU_CASES = [
    ("conv3x3_stride_1_padding_1",
     "--input-channels 16 --output-channels 16 --field {14,14} "
     "--kernel-size 3 --padding 1 --data-type half"),
    ("conv1x1_stride_1",
     "--input-channels 32 --output-channels 16 --field {14,14} "
     "--kernel-size 1 --data-type half --batch-size 2"),
    ("conv_fp32_baseline_config1",
     "--input-channels 16 --output-channels 16 --field {32,32} "
     "--kernel-size 3 --padding 1 --data-type float --bias 0"),
    ("conv3x3_stride_2_float",
     "--input-channels 3 --output-channels 5 --field {9,11} --kernel-size 3 "
     "--stride 2 --padding-lower 1 --padding-upper 0 --data-type float"),
    ("depthwise_5x5",
     "--input-channels 1 --output-channels 1 --conv-groups 24 "
     "--field {28,28} --kernel-size 5 --data-type half"),
    ("conv_zero_batch",
     "--input-channels 4 --output-channels 4 --field {4,4} --kernel-size 3 "
     "--batch-size 0 --data-type half"),
    ("conv_zero_in_chans",
     "--input-channels 0 --output-channels 4 --field {4,4} --kernel-size 3 "
     "--data-type half"),
    ("conv_zero_out_chans",
     "--input-channels 4 --output-channels 0 --field {4,4} --kernel-size 3 "
     "--data-type half"),
    ("conv_negative_padding_via_truncation",
     "--input-channels 8 --output-channels 8 --field {12,12} --kernel-size 3 "
     "--truncation-lower {1,0} --truncation-upper {0,2} --data-type half"),
    ("conv_flips_and_dilation",
     "--input-channels 2 --output-channels 3 --field {7,6} --kernel-size {3,2} "
     "--flip-input {1,0} --flip-kernel {0,1} --in-dilation {2,1} "
     "--kernel-dilation {1,2} --stride {2,2} --data-type float"),
    ("conv_output_padding",
     "--input-channels 2 --output-channels 2 --field {5,5} --kernel-size 2 "
     "--output-padding-lower {1,0} --output-padding-upper {0,2} "
     "--output-truncation-lower {1,1} --data-type float"),
    ("conv_1d_and_3d",
     "--input-channels 8 --output-channels 8 --field {5,6,7} "
     "--kernel-size {2,3,2} --padding {1,0,1} --data-type half"),
    ("conv_quarter_arch_2_AMP",
     "--input-channels 32 --output-channels 16 --field {8,8} --kernel-size 3 "
     "--padding 1 --input-type quarter --output-type half"),
    ("conv_quarter_formats",
     "--input-channels 16 --output-channels 16 --field {6,6} --kernel-size 1 "
     "--input-type quarter --output-type half --fp8-format-fwd quart152 "
     "--fp8-scale-fwd -1 --fp8-scale-weights 3"),
    ("conv_uniform_data_large_accumulation",
     "--input-channels 2048 --output-channels 16 --field {6,6} "
     "--kernel-size 5 --padding 2 --data-type half"),
    ("conv_determinism",
     "--input-channels 16 --output-channels 16 --field {14,14} "
     "--kernel-size 3 --padding 1 --data-type half "
     "--num-determinism-checks 3"),
    ("conv_forced_generic",
     "--input-channels 16 --output-channels 16 --field {14,14} "
     "--kernel-size 3 --padding 1 --data-type half "
     "--fwd-plan-constraints {\"gfx950\":{\"kernel\":\"generic\"}}"),
]


@pytest.mark.gpu
@pytest.mark.parametrize("name,args", GPU_CASES, ids=[c[0] for c in GPU_CASES])
def test_reference_style_cases(name, args):
    print("case", name, flush=True)
    r = run(*args.split())
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert "Validation passed" in r.stdout
    if "large_accumulation" in name:
        assert "Using uniform random data" in r.stdout
    elif "determinism" not in name and "quarter" not in name:
        # (quarter: only 16 contiguous integers, so the reference's rule picks
        # the integer-valued "uniform" mode even for small convolutions)
        assert "no error tolerance" in r.stdout


RANDOM = os.path.join(ROOT, "tests", "tools", "single_conv_layer_random.py")


def test_random_driver_is_reproducible_and_valid():
    """Every emitted parameter set passes ConvParams::validate (via
    --plan-only) and the same seed gives the same command."""
    import sys
    for seed in range(1, 9):
        a = subprocess.run([sys.executable, RANDOM, "--seed", str(seed),
                            "--dry-run"], capture_output=True, text=True)
        b = subprocess.run([sys.executable, RANDOM, "--seed", str(seed),
                            "--dry-run"], capture_output=True, text=True)
        assert a.returncode == 0 and a.stdout == b.stdout
        args = a.stdout.split()[1:]
        r = run(*args, "--plan-only")
        assert r.returncode == 0, (a.stdout, r.stderr)


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(1, 31))
def test_conv_random(seed):
    """conv_random_N of tests/poplin/CMakeLists.txt:1040-1065."""
    import sys
    print("conv_random seed", seed, flush=True)
    r = subprocess.run([sys.executable, RANDOM, "--seed", str(seed)],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(1, 16))
def test_conv_random_quarter(seed):
    import sys
    print("conv_random_quarter seed", seed, flush=True)
    r = subprocess.run([sys.executable, RANDOM, "--seed", str(seed),
                        "--input-type", "quarter"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])


@pytest.mark.gpu
@pytest.mark.parametrize("seed", range(1086, 1106))
def test_conv_random_float(seed):
    # float inputs run on the matrix cores too; these seeds include three
    # field dimensions with output padding and dilated inputs
    import sys
    print("conv_random_float seed", seed, flush=True)
    r = subprocess.run([sys.executable, RANDOM, "--seed", str(seed),
                        "--input-type", "float"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])


# ---------------------------------------------------------------------------
# general_matrix_multiply: the reference's cases for its tool of that name
# (tests/poplin/CMakeLists.txt:515-900).

GEMM = os.path.join(ROOT, "tests", "tools", "general_matrix_multiply")


def gemm(*args, timeout=120):
    if not os.path.exists(GEMM):
        subprocess.check_call(["make", "-C", os.path.dirname(GEMM)],
                              stdout=subprocess.DEVNULL)
    return subprocess.run([GEMM, *args], capture_output=True, text=True,
                          timeout=timeout)


def test_gemm_report_plan_without_a_device():
    r = gemm("--m", "1024", "--k", "512", "--n", "512", "--report-plan",
             "--compile-only")
    assert r.returncode == 0, r.stderr
    assert "implicit GEMM" in r.stdout
    assert "batchSize                  1024" in r.stdout
    # a serial split is an IPU memory device: accepted, and the plan is the
    # unconstrained one
    r2 = gemm("--m", "1024", "--k", "512", "--n", "512", "--report-plan",
              "--compile-only", "--plan-constraints",
              '{"0":{"partition":{"outChanSplit":{"serial":2}}}}')
    assert r2.returncode == 0, r2.stderr
    assert r2.stdout == r.stdout


def test_gemm_usage_errors_exit_1():
    assert gemm("--m", "4", "--k", "4").returncode == 1
    assert gemm("--m", "4", "--k", "4", "--n", "4", "--bogus").returncode == 1
    assert gemm("--m", "4", "--k", "4", "--n", "4", "--left-matrix-op",
                "conjugate").returncode == 1
    r = gemm("--m", "4", "--k", "4", "--n", "4", "--data-type", "half",
             "--input-type", "half", "--output-type", "float")
    assert r.returncode == 1 and "not both" in r.stderr
    r = gemm("--m", "4", "--k", "4", "--n", "4", "--partials-type", "int",
             "--compile-only", "--report-plan")
    assert r.returncode == 1


_OPS = [("normal", "normal"), ("transpose", "normal"), ("normal", "transpose"),
        ("transpose", "transpose")]
GEMM_GPU_CASES = (
    [(f"gemm_{m}x{k}x{n}_{a[:2]}A_{b[:2]}B",
      f"--m {m} --k {k} --n {n} --alpha 1 --beta 1 --tiles-per-ipu=1 "
      f"--left-matrix-op={a} --right-matrix-op={b}")
     for (m, k, n) in ((5, 0, 4), (0, 3, 4), (5, 3, 0)) for a, b in _OPS] + [
        ("gemm_5x0x4_groups3_ignore_data_profile",
         "--g 3 --m 5 --k 0 --n 4 --tiles-per-ipu=1 --ignore-data --profile "
         "--report-plan --show-execution-steps --show-var-storage"),
        ("gemm_1x3x1", "--m 1 --k 3 --n 1 --alpha 1 --beta 1"),
        ("gemm_1x1000x1", "--m 1 --k 1000 --n 1 --alpha 2 --beta 1"),
        ("gemm_40x40x40", "--m 40 --k 40 --n 40 --alpha 2 --beta 1"),
        ("gemm_10x20x30_groups5",
         "--g 5 --m 10 --k 20 --n 30 --alpha 2 --beta 3"),
        ("gemm_40x39x38", "--m 40 --k 39 --n 38 --alpha 2 --beta 1"),
        ("gemm_40x39x38_left_transpose",
         "--m 40 --k 39 --n 38 --alpha 2 --beta 1 --left-matrix-op=transpose"),
        ("gemm_40x39x38_right_transpose",
         "--m 40 --k 39 --n 38 --alpha 2 --beta 1 "
         "--right-matrix-op=transpose"),
        ("gemm_40x40x40_halffloat",
         "--m 40 --k 40 --n 40 --alpha 2 --beta 1 --input-type=half "
         "--output-type=float"),
        ("gemm_40x39x38_floathalf",
         "--m 40 --k 39 --n 38 --alpha 2 --beta 1 --input-type=float "
         "--output-type=half"),
        ("gemm_40x39x38_right_transpose_floathalf",
         "--m 40 --k 39 --n 38 --alpha 2 --beta 1 --right-matrix-op=transpose "
         "--input-type=float --output-type=half"),
        ("gemm_100x100x100_serial_split_nx2",
         "--m 100 --k 100 --n 100 --plan-constraints "
         '{"0":{"partition":{"outChanSplit":{"serial":2}}}}'),
        ("gemm_float_40x39x38", "--m 40 --k 39 --n 38 --data-type float"),
        # matrix-core and streaming kernels, tighter tolerance than the
        # tool's default 10 % for half
        ("gemm_1024x512x512_mfma",
         "--m 1024 --k 512 --n 512 --alpha 1 --beta 0 --tolerance 0.01"),
        ("gemm_groups4_300x72x136_mfma",
         "--g 4 --m 300 --k 72 --n 136 --input-type=half --output-type=float "
         "--tolerance 0.01"),
        ("gemm_4100x256x64_pointwise",
         "--m 4100 --k 256 --n 64 --input-type=half --output-type=float "
         "--tolerance 0.01 --use-create-output=true"),
        ("gemm_prearranged_rhs_repeated",
         "--m 700 --k 136 --n 72 --input-type=half --output-type=float "
         "--tolerance 0.01 --pre-arrange-rhs=true --num-executions 3"),
        ("gemm_quarter",
         "--m 200 --k 256 --n 128 --input-type=quarter --output-type=half "
         "--fp8-format-a quart143 --fp8-format-b quart143 --fp8-scale-b -2"),
    ])


@pytest.mark.gpu
@pytest.mark.parametrize("name,args", GEMM_GPU_CASES,
                         ids=[c[0] for c in GEMM_GPU_CASES])
def test_gemm_reference_cases(name, args):
    r = gemm(*args.split())
    assert r.returncode == 0, (name, r.stdout[-2000:], r.stderr[-2000:])


C2_ARGS = ("--input-channels 128 --output-channels 128 --field {28,28} "
           "--kernel-size 3 --padding 1 --batch-size 32 --data-type half "
           "--bias 0").split()


@pytest.mark.gpu
def test_test_planner_compares_estimates_with_measurements():
    """--test-planner (tools/single_conv_layer.cpp:183, 857-888, 1490-1520):
    every pass's planner estimate against the time between two HIP events;
    within the stated factor on the benchmark's 3x3 layer, and a failure
    when the tolerance is made impossible."""
    r = run(*C2_ARGS, "--test-planner", timeout=300)
    assert r.returncode == 0, (r.stdout[-3000:], r.stderr[-3000:])
    import re
    rows = dict((m[0], (float(m[1]), float(m[2]))) for m in re.findall(
        r"^  (fwd|bwd|wu): estimated ([0-9.]+) us, measured ([0-9.]+) us",
        r.stdout, re.M))
    assert set(rows) == {"fwd", "bwd", "wu"}, r.stdout
    for est, measured in rows.values():
        assert measured <= 2.5 * est + 15 and est <= 2.5 * measured + 15
    bad = run(*C2_ARGS, "--test-planner", "--test-planner-tolerance", "0.001",
              "--single-phase", "wu", timeout=300)
    assert bad.returncode == 1 and "beyond the tolerance" in bad.stdout


@pytest.mark.gpu
def test_tensor_files_chain_two_layers(tmp_path):
    """--fwd-out-file of one run is --fwd-in-file of the next, whose batch
    size, field and type come from the file
    (tools/single_conv_layer.cpp:418-429, 593-626, 1376-1382)."""
    first = str(tmp_path / "layer1.bin")
    r = run("--input-channels", "16", "--output-channels", "32", "--field",
            "{12,10}", "--kernel-size", "3", "--padding", "1", "--batch-size",
            "3", "--data-type", "half", "--single-phase", "fwd",
            "--fwd-out-file", first)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert "Saving FWD tensor with shape:[3,32,12,10]" in r.stdout
    second = str(tmp_path / "layer2.bin")
    r = run("--input-channels", "32", "--output-channels", "8",
            "--kernel-size", "{1,3}", "--single-phase", "fwd",
            "--fwd-in-file", first, "--fwd-out-file", second,
            "--tolerance", "0.02")
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert "Importing FWD input from file, shape:[3,32,12,10]" in r.stdout
    assert "Saving FWD tensor with shape:[3,8,12,8]" in r.stdout
    # the options the file replaces may not be given beside it
    r = run("--input-channels", "32", "--output-channels", "8", "--field",
            "{12,10}", "--fwd-in-file", first)
    assert r.returncode == 1 and "Cannot specify --field" in r.stderr
    r = run("--input-channels", "31", "--output-channels", "8",
            "--fwd-in-file", first)
    assert r.returncode == 1 and "dimension 1" in r.stderr
    r = run("--input-channels", "32", "--output-channels", "8",
            "--fwd-in-file", str(tmp_path / "missing.bin"))
    assert r.returncode == 1 and "could not be opened" in r.stderr
    # the backward pass's input and output likewise
    grads = str(tmp_path / "grads.bin")
    r = run("--input-channels", "8", "--output-channels", "32", "--field",
            "{12,10}", "--kernel-size", "3", "--padding", "1", "--batch-size",
            "3", "--single-phase", "bwd", "--bwd-in-file", first,
            "--bwd-out-file", grads, "--tolerance", "0.05")
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert "Importing BWD input from file, shape:[3,32,12,10]" in r.stdout
    assert "Saving BWD tensor with shape:[3,8,12,10]" in r.stdout


@pytest.mark.gpu
def test_create_output_and_generic_input_layout():
    """--use-create-output=true (tools/single_conv_layer.cpp:407) and
    --use-create-input=false (an input in the plan-independent layout)."""
    for extra in (["--use-create-output=true"], ["--use-create-input=false"],
                  ["--use-create-output=true", "--use-create-input=false",
                   "--single-phase=all"]):
        r = run("--input-channels", "64", "--output-channels", "64", "--field",
                "{14,14}", "--kernel-size", "3", "--padding", "1",
                "--batch-size", "4", *extra)
        assert r.returncode == 0, (extra, r.stdout[-2000:], r.stderr[-2000:])
        assert "Validation passed" in r.stdout


@pytest.mark.gpu
def test_backward_fp8_metadata_and_per_pass_constraint_files(tmp_path):
    """--fp8-format-bwd / --fp8-scale-bwd describe the backward pass's input;
    --bwd-plan-constraints-file / --wu-plan-constraints-file give a pass its
    own constraints."""
    base = ["--input-channels", "32", "--output-channels", "32", "--field",
            "{10,10}", "--kernel-size", "3", "--padding", "1", "--batch-size",
            "2", "--input-type", "quarter", "--output-type", "half"]
    for fmt, scale in (("quart143", "-1"), ("quart152", "3")):
        r = run(*base, "--single-phase", "bwd", "--fp8-format-bwd", fmt,
                "--fp8-scale-bwd", scale)
        assert r.returncode == 0, (fmt, r.stdout[-2000:], r.stderr[-2000:])
    assert run(*base, "--fp8-format-bwd", "quart8").returncode == 1
    generic = tmp_path / "generic.json"
    generic.write_text('{"gfx950": {"kernel": "generic"}}')
    half = ["--input-channels", "32", "--output-channels", "32", "--field",
            "{10,10}", "--kernel-size", "3", "--padding", "1", "--batch-size",
            "2", "--report-plan", "1"]
    r = run(*half, "--bwd-plan-constraints-file", str(generic),
            "--wu-plan-constraints-file", str(generic))
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    fwd, rest = r.stdout.split("Backward plan:")
    bwd, wu = rest.split("WU plan:")
    assert "implicit GEMM" in fwd and "generic direct" not in fwd
    assert "generic direct" in bwd and "generic direct" in wu
    r = run(*half, "--bwd-plan-constraints-file", str(generic),
            "--bwd-plan-constraints", '{"gfx950": {"kernel": "igemm"}}')
    assert r.returncode == 1 and "Both bwd-plan-constraints" in r.stderr


@pytest.mark.gpu
def test_gemm_prearranged_for_another_kernel_is_refused():
    """A right-hand side arranged for the streaming matrix-core kernel has the
    byte count of one arranged for the 1x1 kernel (k = 256, n = 64) but
    another operand order: the multiplication must refuse it, not read it."""
    base = ("--m 4100 --k 256 --n 64 --input-type=half --output-type=float "
            "--tolerance 0.01 --pre-arrange-rhs=true").split()
    ok = gemm(*base)
    assert ok.returncode == 0, (ok.stdout[-2000:], ok.stderr[-2000:])
    r = gemm(*base, "--pre-arrange-plan-constraints",
             '{"gfx950":{"kernel":"igemm"}}')
    assert r.returncode == 1, (r.stdout[-2000:], r.stderr[-2000:])
    assert "arranged" in r.stderr + r.stdout


# ---------------------------------------------------------------------------
# multi_conv_layer: the reference's cases for its tool of that name
# (tests/poplin/CMakeLists.txt:4019-4069), --conv arguments from the same JSON
# documents.

MULTI = os.path.join(ROOT, "tests", "tools", "multi_conv_layer")


def _golden(name):
    with open(os.path.join(ROOT, "tests", "golden", name)) as f:
        return f.read()


def multi(*args, timeout=120):
    if not os.path.exists(MULTI):
        subprocess.check_call(["make", "-C", os.path.dirname(MULTI)],
                              stdout=subprocess.DEVNULL)
    return subprocess.run([MULTI, *args], capture_output=True, text=True,
                          timeout=timeout)


def test_multi_conv_layer_plans_without_a_device():
    r = multi("--conv", _golden("depthwise_conv_half.json"), "--conv",
              _golden("pointwise_conv_float.json"), "--report-plan", "1",
              "--compile-only")
    assert r.returncode == 0, r.stderr
    assert "got 2 convs" in r.stdout
    assert r.stdout.count("Plan:") == 2
    assert "depthwise direct" in r.stdout
    r = multi("--conv", _golden("depthwise_conv_half.json"),
              "--multiconv-options", '{"planType": "diagonal"}')
    assert r.returncode == 1 and "planType" in r.stderr
    assert multi("--conv", "{not json").returncode == 1


MULTI_GPU_CASES = [
    ("multi_conv_different_types",
     ["depthwise_conv_half.json", "pointwise_conv_float.json"], []),
    ("multi_conv_different_types_single_tile",
     ["depthwise_conv_half.json", "depthwise_conv_half.json"],
     ["--tiles-per-ipu", "1"]),
    ("multi_conv_different_types_bwd",
     ["depthwise_conv_half.json", "pointwise_reusable_conv_float.json"],
     ["--bwd", "1", "--enable-convolution-reuse", "0"]),
    ("multi_conv_different_types_bwd_reuse",
     ["depthwise_conv_half.json", "pointwise_reusable_conv_float.json"],
     ["--bwd", "1", "--enable-convolution-reuse", "1"]),
    ("multi_conv_quarter_half_fwd",
     ["depthwise_conv_quarter1.json", "depthwise_conv_quarter2.json"],
     ["--bwd", "0"]),
    ("multi_conv_quarter_half_bwd",
     ["depthwise_conv_quarter1.json", "depthwise_conv_quarter2.json"],
     ["--bwd", "1"]),
    ("multi_conv_serial_five",
     ["depthwise_conv_half.json", "pointwise_conv_float.json",
      "pointwise_reusable_conv_float.json", "depthwise_conv_half.json",
      "pointwise_conv_float.json"],
     ["--multiconv-options", '{"planType": "serial"}']),
    ("multi_conv_parallel_five",
     ["depthwise_conv_half.json", "pointwise_conv_float.json",
      "pointwise_reusable_conv_float.json", "depthwise_conv_half.json",
      "pointwise_conv_float.json"], []),
]


@pytest.mark.gpu
@pytest.mark.parametrize("name,convs,extra", MULTI_GPU_CASES,
                         ids=[c[0] for c in MULTI_GPU_CASES])
def test_multi_conv_reference_cases(name, convs, extra):
    args = []
    for c in convs:
        args += ["--conv", _golden(c)]
    r = multi(*args, *extra)
    assert r.returncode == 0, (name, r.stdout[-2000:], r.stderr[-2000:])
    assert "Validation passed" in r.stdout

"""The reference's whole ctest matrix for its `single_conv_layer` tool (and, at
the end of this file, for `general_matrix_multiply`), carried
as a fixture: every add_multitarget_test(... COMMAND single_conv_layer ...) of
tests/poplin/CMakeLists.txt:986-3500 with its foreach loops expanded
(tests/golden/single_conv_layer_ctest_matrix.json, written by
tests/golden/extract_ctest_matrix.py; 183 source invocations, 537 argument
lists).  On the GPU all of them run through this build's harness - forward,
backward and weight update passes as the arguments say - and the harness's
own comparison with the host model decides (exit code 0; these cases use +-1
data, so the comparison is exact).  IPU-only arguments (--tiles-per-ipu,
--ipus, IPU plan constraints such as AMP / SLIC methods and tile partitions)
are validated and then have no effect, or map to the gfx950 kernel that has
the method's role.  All 537 run in one process (--batch-file)."""
import json
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "tests", "tools", "single_conv_layer")
GOLDEN = os.path.join(ROOT, "tests", "golden")

with open(os.path.join(GOLDEN, "single_conv_layer_ctest_matrix.json")) as _f:
    MATRIX = json.load(_f)["tests"]
NAMES = [t["name"] for t in MATRIX]

# Options of the reference tool (tools/single_conv_layer.cpp:171-430).
REFERENCE_OPTIONS = {
    "help", "compile-only", "device-type", "profile", "profile-dir",
    "test-planner", "test-planner-existing-profile",
    "test-planner-simulated-execution-file", "test-planner-report-all-tiles",
    "test-planner-report-all-serial-splits", "test-planner-report-verbose",
    "test-planner-print-vars", "ignore-data", "input-channels",
    "output-channels", "field", "kernel-size", "bias", "data-type",
    "input-type", "output-type", "fp8-scale-fwd", "fp8-scale-weights",
    "fp8-scale-bwd", "fp8-format-fwd", "fp8-format-weights", "fp8-format-bwd",
    "truncation", "truncation-upper", "truncation-lower", "in-dilation",
    "padding", "padding-upper", "padding-lower", "flip-input",
    "kernel-truncation", "kernel-truncation-upper", "kernel-truncation-lower",
    "kernel-dilation", "kernel-padding", "kernel-padding-upper",
    "kernel-padding-lower", "flip-kernel", "output-truncation",
    "output-truncation-upper", "output-truncation-lower", "stride",
    "output-padding", "output-padding-upper", "output-padding-lower",
    "single-phase", "plan-only", "inference-only", "tolerance",
    "absolute-tolerance", "ipus", "tiles-per-ipu", "input-load-width",
    "workers-per-tile", "batch-size", "conv-groups", "fwd-plan-constraints",
    "fwd-plan-constraints-file", "bwd-plan-constraints",
    "bwd-plan-constraints-file", "wu-plan-constraints",
    "wu-plan-constraints-file", "report-plan", "report-var-storage",
    "remap-output-tensor", "enable-convolution-reuse", "convolution-options",
    "use-create-input", "use-create-output", "num-determinism-checks",
    "preplan", "fwd-in-file", "fwd-out-file", "bwd-in-file", "bwd-out-file"}


def _options_of(args):
    return {a[2:].split("=", 1)[0] for a in args if a.startswith("--")}


def test_fixture_is_the_whole_matrix():
    assert len(MATRIX) == 537
    assert len({t["line"] for t in MATRIX}) == 183
    assert len(set(NAMES)) == len(NAMES)
    used = set().union(*(_options_of(t["args"]) for t in MATRIX))
    assert used <= REFERENCE_OPTIONS, used - REFERENCE_OPTIONS
    # the passes the matrix exercises
    phases = [next((a.split("=", 1)[1] for a in t["args"]
                    if a.startswith("--single-phase=")), None)
              for t in MATRIX]
    assert {"fwd", "bwd", "wu", "all"} <= set(phases) | {"all"}
    # plan-constraint files travel with the fixture
    for t in MATRIX:
        for a in t["args"]:
            if "@golden/" in a:
                assert os.path.exists(
                    os.path.join(GOLDEN, a.split("@golden/", 1)[1]))


def test_every_reference_option_is_accepted(tmp_path):
    """No option of the reference tool is an unknown option here (an option's
    value may still be refused)."""
    src = open(os.path.join(ROOT, "tests", "tools",
                            "single_conv_layer.cpp")).read()
    known = set(re.findall(r'"([a-z0-9-]+)"',
                           src.split("static const char *known[]", 1)[1]
                           .split("};", 1)[0]))
    assert REFERENCE_OPTIONS <= known, REFERENCE_OPTIONS - known


@pytest.fixture(scope="session")
def matrix_results(tmp_path_factory):
    if not os.path.exists(TOOL):
        subprocess.check_call(["make", "-C", os.path.dirname(TOOL)],
                              stdout=subprocess.DEVNULL)
    cases = [{"name": t["name"],
              "args": [a.replace("@golden/", GOLDEN + "/") for a in t["args"]]}
             for t in MATRIX]
    batch = tmp_path_factory.mktemp("matrix") / "cases.json"
    batch.write_text(json.dumps(cases))
    r = subprocess.run([TOOL, "--batch-file", str(batch)],
                       capture_output=True, text=True, timeout=900)
    out, results = {}, {}
    name = None
    for line in r.stdout.splitlines():
        if line.startswith("### CASE "):
            name = line[9:]
            out[name] = []
        elif line.startswith("### RESULT "):
            n, rc = line[11:].rsplit(" ", 1)
            results[n] = int(rc)
            name = None
        elif name is not None:
            out[name].append(line)
    return results, out, r


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_reference_ctest_case(matrix_results, name):
    results, out, r = matrix_results
    assert name in results, (r.returncode, r.stdout[-1500:], r.stderr[-1500:])
    text = "\n".join(out[name])
    assert results[name] == 0, text[-3000:]
    assert "Validation passed" in text


# ---------------------------------------------------------------------------
# general_matrix_multiply: the 39 invocations of the same CMakeLists.txt
# (:519-985), through this build's tool of that name.  The tool compares with
# a host matrix product itself; plan constraints written for the IPU planner
# (serial splits of the output or input channels) are validated and have no
# effect here.

GEMM_TOOL = os.path.join(ROOT, "tests", "tools", "general_matrix_multiply")
with open(os.path.join(GOLDEN,
                       "general_matrix_multiply_ctest_matrix.json")) as _f:
    GEMM_MATRIX = json.load(_f)["tests"]

# Options of the reference tool (tools/general_matrix_multiply.cpp:120-225).
GEMM_REFERENCE_OPTIONS = {
    "help", "compile-only", "device-type", "profile", "profile-dir",
    "ignore-data", "m", "k", "n", "g", "data-type", "input-type",
    "output-type", "partials-type", "fp8-scale-A", "fp8-scale-B",
    "fp8-format-A", "fp8-format-B", "alpha", "beta", "left-matrix-op",
    "right-matrix-op", "tolerance", "tiles-per-ipu",
    "available-memory-proportion", "enable-fast-reduce", "report-plan",
    "show-execution-steps", "show-var-storage", "ipus", "plan-constraints",
    "num-executions", "remap-output-tensor", "plan-constraints-file",
    "use-create-output"}


def test_gemm_fixture_is_the_whole_matrix():
    assert len(GEMM_MATRIX) == 39
    assert len({t["name"] for t in GEMM_MATRIX}) == 39
    used = set().union(*(_options_of(t["args"]) for t in GEMM_MATRIX))
    assert used <= GEMM_REFERENCE_OPTIONS, used - GEMM_REFERENCE_OPTIONS
    # ... and this build's tool knows every one of the reference's options
    src = open(os.path.join(ROOT, "tests", "tools",
                            "general_matrix_multiply.cpp")).read()
    known = set(re.findall(r'"([A-Za-z0-9-]+)"',
                           src.split("static const char *known[]", 1)[1]
                           .split("};", 1)[0]))
    assert GEMM_REFERENCE_OPTIONS <= known, GEMM_REFERENCE_OPTIONS - known
    # empty operands, transposed operands, groups, mixed types, quarter
    text = " ".join(" ".join(t["args"]) for t in GEMM_MATRIX)
    for needle in ("--k 0", "--m 0", "--left-matrix-op=transpose",
                   "--right-matrix-op=transpose", "--g 5",
                   "--input-type=quarter", "--use-create-output=true"):
        assert needle in text


@pytest.mark.gpu
@pytest.mark.parametrize("case", GEMM_MATRIX, ids=lambda t: t["name"])
def test_reference_gemm_ctest_case(case):
    if not os.path.exists(GEMM_TOOL):
        subprocess.check_call(["make", "-C", os.path.dirname(GEMM_TOOL)],
                              stdout=subprocess.DEVNULL)
    args = [a.replace("@golden/", GOLDEN + "/") for a in case["args"]]
    r = subprocess.run([GEMM_TOOL, *args], capture_output=True, text=True,
                       timeout=120)
    # (the tool, like the reference's, says nothing when the product matches
    # the host model and exits with 1 and "Validation failed" when it does not)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert "Validation failed" not in r.stderr

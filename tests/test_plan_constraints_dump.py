"""planConstraintsOutputFilename and the plan's constraints document: the
dump, given back as planConstraints, must reproduce the plan exactly
(reference: include/poplin/Convolution.hpp:191-199,
lib/poplin/ConvPlan.cpp:1574-1666, 1764; the reference's own round-trip test is
tests/poplin/ConvPlanTest.cpp:121-175).  No GPU needed: planning is host work."""
import json
import os

import pytest

import poplibs_amd as pa
from helpers import make_params

H, Q, F = pa.HALF, pa.QUARTER, pa.FLOAT

LAYERS = {
    "c2_patch16": make_params(H, batch=32, field=(28, 28), kernel=(3, 3),
                              ci=128, co=128, pad=1),
    "c3_pointwise": make_params(H, batch=32, field=(56, 56), kernel=(1, 1),
                                ci=256, co=64),
    "c4_rows": make_params(H, batch=32, field=(112, 112), kernel=(3, 3),
                           groups=96, stride=2, pad=1),
    "c5_fp8_patch16": make_params(Q, H, batch=64, field=(14, 14),
                                  kernel=(3, 3), ci=256, co=256, pad=1),
    "c1_fp32": make_params(F, batch=1, field=(32, 32), kernel=(3, 3), ci=16,
                           co=16, pad=1),
    "split_k": make_params(H, batch=32, field=(7, 7), kernel=(3, 3), ci=512,
                           co=512, pad=1),
    "patch32": make_params(H, batch=8, field=(28, 28), kernel=(3, 3), ci=128,
                           co=128, pad=1),
    "strided_3x3": make_params(H, batch=32, field=(56, 56), kernel=(3, 3),
                               ci=128, co=128, pad=1, stride=2),
    "pointwise_widening": make_params(H, batch=32, field=(56, 56),
                                      kernel=(1, 1), ci=64, co=256),
    "pointwise_512": make_params(H, batch=32, field=(14, 14), kernel=(1, 1),
                                 ci=1024, co=256),
    "two_stage_tiles": make_params(H, batch=64, field=(56, 56), kernel=(3, 3),
                                   ci=96, co=128, pad=1),
    "depthwise_small": make_params(H, batch=2, field=(14, 14), kernel=(3, 3),
                                   groups=64, pad=1),
    "depthwise_7x7": make_params(H, batch=4, field=(28, 28), kernel=(7, 7),
                                 groups=32, pad=3),
    "depthwise_5x5": make_params(H, batch=32, field=(56, 56), kernel=(5, 5),
                                 groups=144, pad=2, stride=2),
    "generic_flip": make_params(H, batch=2, field=(9, 9), kernel=(3, 3), ci=8,
                                co=8, flipIn=[True, False]),
    "grouped": make_params(H, batch=16, field=(28, 28), kernel=(3, 3), ci=32,
                           co=32, groups=4, pad=1),
    "grouped_wide": make_params(H, batch=16, field=(28, 28), kernel=(3, 3),
                                ci=64, co=128, groups=2, pad=1),
    "groups_as_one": make_params(H, batch=16, field=(28, 28), kernel=(3, 3),
                                 ci=4, co=4, groups=32, pad=1),
}


def _tiling(plan):
    """Everything of the plan report except the parameters, the reason line
    and the list of tilings weighed (a forced plan weighs none)."""
    lines = plan.describe().split("Plan (gfx950", 1)[1].splitlines()
    keep, skipping = [], False
    for line in lines:
        head = line.strip().split("  ")[0]
        if head == "tilings weighed":
            skipping = True
            continue
        if skipping and (line.startswith("            ")
                         or line.startswith("          *")):
            continue
        skipping = False
        if head != "reason":
            keep.append(line)
    return "\n".join(keep)


@pytest.mark.parametrize("name", sorted(LAYERS))
def test_constraints_reproduce_the_plan(name):
    p = LAYERS[name]
    plan = pa.Plan(p)
    text = plan.constraints()
    doc = json.loads(text)
    # (layers of several conv groups on the matrix cores also say how many
    # groups run as one)
    assert list(doc) in (["gfx950"], ["convGroupsPerGroup", "gfx950"])
    assert "kernel" in doc["gfx950"]
    again = pa.Plan(p, {"planConstraints": text})
    assert _tiling(again) == _tiling(plan)
    assert plan.packs_like(again) and again.packs_like(plan)
    for which in range(6):
        assert plan.buffer_bytes(which) == again.buffer_bytes(which)
    # a fixed point: the forced plan dumps the same document
    assert again.constraints() == text


def test_constraints_pin_the_plan_against_the_planners_choice():
    """The dump of a plan that is NOT the planner's choice still reproduces
    that plan, not the choice."""
    p = LAYERS["c2_patch16"]
    forced = pa.Plan(p, {"planConstraints": '{"gfx950": {"patch": 0}}'})
    assert "resident" not in forced.describe().split("tilings weighed")[0]
    again = pa.Plan(p, {"planConstraints": forced.constraints()})
    assert _tiling(again) == _tiling(forced)
    assert not again.packs_like(pa.Plan(p))


@pytest.mark.parametrize("pass_,suffix", [
    ("TRAINING_FWD", "_FWD"), ("INFERENCE_FWD", "_FWD"),
    ("TRAINING_BWD", "_BWD"), ("FC_TRAINING_BWD", "_BWD"),
    ("TRAINING_WU", "_WU"), ("NONE", ""), (None, "")])
def test_output_filename_by_pass(tmp_path, pass_, suffix):
    p = LAYERS["c2_patch16"]
    base = str(tmp_path / "plan")
    opts = {"planConstraintsOutputFilename": base}
    if pass_:
        opts["pass"] = pass_
    plan = pa.Plan(p, opts)
    path = base + suffix + ".json"
    assert os.listdir(tmp_path) == [os.path.basename(path)]
    with open(path) as f:
        text = f.read()
    assert json.loads(text) == json.loads(plan.constraints())
    back = {"planConstraints": text.strip()}
    if pass_:
        back["pass"] = pass_
    again = pa.Plan(p, back)
    assert _tiling(again) == _tiling(plan)


def test_weight_update_plan_writes_the_wu_file(tmp_path):
    p = LAYERS["c2_patch16"]
    base = str(tmp_path / "layer")
    plan = pa.WeightUpdatePlan(p, {"planConstraintsOutputFilename": base,
                                   "pass": "TRAINING_FWD"})
    assert os.listdir(tmp_path) == ["layer_WU.json"]
    with open(base + "_WU.json") as f:
        text = f.read().strip()
    assert json.loads(text) == json.loads(plan.constraints())
    assert json.loads(text)["gfx950"]["weightDeltas"] == 1
    again = pa.WeightUpdatePlan(p, {"planConstraints": text})
    assert _tiling(again) == _tiling(plan)
    assert again.workspace_bytes() == plan.workspace_bytes()
    # ... and the pass through its own convolution, by name
    conv = pa.WeightUpdatePlan(
        p, {"planConstraints": '{"gfx950": {"weightDeltas": 0}}'})
    assert "as a weight update pass" not in conv.describe()
    assert json.loads(conv.constraints())["gfx950"]["weightDeltas"] == 0
    conv2 = pa.WeightUpdatePlan(p, {"planConstraints": conv.constraints()})
    assert _tiling(conv2) == _tiling(conv)


@pytest.mark.parametrize("name", ["c4_rows", "depthwise_small", "grouped",
                                  "grouped_wide", "c2_patch16"])
def test_weight_update_constraints_round_trip(name):
    p = LAYERS[name]
    plan = pa.WeightUpdatePlan(p)
    again = pa.WeightUpdatePlan(p, {"planConstraints": plan.constraints()})
    assert _tiling(again) == _tiling(plan)
    assert again.workspace_bytes() == plan.workspace_bytes()
    assert again.constraints() == plan.constraints()


def test_small_grouped_layer_keeps_the_general_weight_update_path():
    """In a grouped layer every group brings its own 128 x 128 tiles per tap
    to the matrix-core weight-delta kernel: where the channels fill no more
    than a quarter of a tile (measured: 32 groups of 16 -> 16 channels 420 us
    against 117 us, 4 groups of 64 -> 64 41 against 34), the planner leaves
    the layer to the pass's own convolution unless the kernel is asked for by
    name."""
    def picks(**kw):
        p = make_params(H, batch=32, field=(28, 28), kernel=(3, 3), pad=1, **kw)
        return "matrix-core weight-delta" in pa.WeightUpdatePlan(p).describe()
    assert not picks(ci=16, co=16, groups=32)
    assert not picks(ci=32, co=32, groups=8)
    assert not picks(ci=64, co=64, groups=2)
    assert picks(ci=64, co=128, groups=2)
    assert picks(ci=16, co=16)
    assert picks(ci=32, co=64)
    p = make_params(H, batch=32, field=(28, 28), kernel=(3, 3), ci=16, co=16,
                    groups=32, pad=1)
    forced = pa.WeightUpdatePlan(
        p, {"planConstraints": '{"gfx950": {"weightDeltas": 1}}'})
    assert "matrix-core weight-delta" in forced.describe()

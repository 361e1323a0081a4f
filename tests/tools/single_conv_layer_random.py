#!/usr/bin/env python3
"""Seeded random-parameter driver for the single_conv_layer harness.

Test infrastructure.  Draws one convolution from the same ranges and
distributions as the reference's fuzz driver
(tools/single_conv_layer_random.py:38-56 bounds, :213-370 distributions,
:372-395 validity / FLOP filter) - up to 8 groups, batch up to 16, 2-3 field
dimensions up to 256, input dilation up to 4, padding up to 5, kernels up to
16 with dilation up to 4 and padding up to 3, strides up to 4, truncated
geometric weights favouring small values, 30 % "symmetrical" convolutions
(output shape == input shape) - and runs the harness on it, which checks the
GPU result against the host model.  The random stream is this script's own
(`random.Random(seed)`); reproducing the reference's stream is not a goal.

    single_conv_layer_random.py --seed 7 [--input-type half|float|quarter|all]
"""
import argparse
import os
import random
import subprocess
import sys
from bisect import bisect_left
from functools import reduce
from operator import mul

HERE = os.path.dirname(os.path.abspath(__file__))

VECTOR_WIDTH = {"quarter": 8, "half": 4, "float": 2}
AMP_IN_CHANS = {"quarter": 32, "half": 16, "float": 4}
MAX_CONV_GROUPS = 8
MAX_BATCH_SIZE = 16
MIN_FIELD_DIMS, MAX_FIELD_DIMS = 2, 3
MAX_FIELD_SIZE = 256
MAX_IN_DILATION = 4
MAX_PADDING = 5
MAX_KERNEL_SIZE = 16
MAX_KERNEL_DILATION = 4
MAX_KERNEL_PADDING = 3
MAX_CHANS_PER_GROUP = 512
MAX_STRIDE = 4


def weighted_choice(rng, seq, weights):
    cumulative, total = [], 0.0
    for _, w in zip(seq, weights):
        total += w
        cumulative.append(total)
    return seq[bisect_left(cumulative, rng.uniform(0, total))]


def geometric_choice(rng, seq, ratio):
    """Element i is picked with weight ratio**i (truncated geometric)."""
    seq = list(seq)
    return weighted_choice(rng, seq, [ratio ** i for i in range(len(seq))])


class Params:
    pass


def make_params(rng, input_type):
    p = Params()
    symmetrical = rng.randrange(0, 100) > 70
    if input_type == "float":
        types = [("float", "float")]
    elif input_type == "half":
        types = [("half", "half")]
    elif input_type == "quarter":
        types = [("quarter", "half")]
    else:
        types = [("float", "float"), ("half", "half")]
    if not symmetrical and input_type in ("all", "half"):
        types.append(("half", "float"))   # (data type, partials type)
    p.data_type, p.partials_type = rng.choice(types)
    p.batch_size = geometric_choice(rng, range(1, MAX_BATCH_SIZE + 1), 0.4)
    p.conv_groups = geometric_choice(rng, range(1, MAX_CONV_GROUPS + 1), 0.4)

    def chans():
        multiple = weighted_choice(
            rng, [1, VECTOR_WIDTH[p.data_type], AMP_IN_CHANS[p.data_type]],
            [0.25, 0.25, 0.5]) * p.conv_groups
        return geometric_choice(
            rng, range(1, MAX_CHANS_PER_GROUP // multiple + 1),
            0.9 ** multiple) * multiple

    p.in_chans = chans()
    p.out_chans = p.in_chans if symmetrical else chans()
    dims = rng.randrange(MIN_FIELD_DIMS, MAX_FIELD_DIMS + 1)
    p.field = [geometric_choice(rng, range(1, MAX_FIELD_SIZE + 1), 0.9)
               for _ in range(dims)]
    p.stride = [geometric_choice(rng, range(1, MAX_STRIDE + 1), 0.5)
                for _ in range(dims)]
    p.pad_lower, p.pad_upper, p.in_dilation = [], [], []
    for i in range(dims):
        lowest = 1
        if symmetrical:
            # out == in needs k = x - x s + p + s > 0 with x the dilated size
            s = p.stride[i]
            x = p.field[i] + (s - 1) * (p.field[i] - 1)
            lowest = x * s - x - s + 1
        p.pad_lower.append(geometric_choice(
            rng, range(lowest, max(lowest, MAX_PADDING) + 1), 0.5))
        if symmetrical:
            p.pad_upper.append(p.pad_lower[i])
            p.in_dilation.append(p.stride[i])
        else:
            p.pad_upper.append(
                geometric_choice(rng, range(1, MAX_PADDING + 1), 0.5))
            p.in_dilation.append(
                geometric_choice(rng, range(1, MAX_IN_DILATION + 1), 0.5))
    p.kernel, p.k_pad_lower, p.k_pad_upper, p.k_dilation = [], [], [], []
    for i in range(dims):
        if symmetrical:
            s = p.stride[i]
            x = p.field[i] + (s - 1) * (p.field[i] - 1)
            k = x - x * s + p.pad_lower[i] + p.pad_upper[i] + s
            assert k > 0
            p.kernel.append(k)
            p.k_pad_lower.append(0)
            p.k_pad_upper.append(0)
            p.k_dilation.append(1)
        else:
            p.kernel.append(
                geometric_choice(rng, range(1, MAX_KERNEL_SIZE + 1), 0.7))
            p.k_pad_lower.append(
                geometric_choice(rng, range(0, MAX_KERNEL_PADDING + 1), 0.3))
            p.k_pad_upper.append(
                geometric_choice(rng, range(0, MAX_KERNEL_PADDING + 1), 0.3))
            p.k_dilation.append(
                geometric_choice(rng, range(1, MAX_KERNEL_DILATION + 1), 0.5))
    return p


def transformed(shape, dilation, lower, upper):
    return [lo + (1 + (s - 1) * d if s else 0) + up
            for s, d, lo, up in zip(shape, dilation, lower, upper)]


def flops(p):
    tin = transformed(p.field, p.in_dilation, p.pad_lower, p.pad_upper)
    tk = transformed(p.kernel, p.k_dilation, p.k_pad_lower, p.k_pad_upper)
    out = [(i - k) // s + 1 for i, k, s in zip(tin, tk, p.stride)]
    return 2 * (reduce(mul, out, 1) * p.conv_groups * p.batch_size
                * reduce(mul, p.kernel, 1) * p.in_chans * p.out_chans)


def make_constrained_params(rng, input_type, max_flops, max_elems):
    while True:
        p = make_params(rng, input_type)
        tin = transformed(p.field, p.in_dilation, p.pad_lower, p.pad_upper)
        tk = transformed(p.kernel, p.k_dilation, p.k_pad_lower, p.k_pad_upper)
        if any(i < k for i, k in zip(tin, tk)):
            continue
        if flops(p) > max_flops:
            continue
        # keep the host model's staging arrays small
        if (reduce(mul, tin, 1) * p.batch_size * p.in_chans * p.conv_groups
                > max_elems):
            continue
        return p


def braces(values):
    return "{" + ",".join(str(v) for v in values) + "}"


def command(p, binary):
    cmd = [binary,
           "--input-channels", str(p.in_chans),
           "--output-channels", str(p.out_chans),
           "--conv-groups", str(p.conv_groups),
           "--batch-size", str(p.batch_size),
           "--field", braces(p.field),
           "--kernel-size", braces(p.kernel),
           "--stride", braces(p.stride),
           "--padding-lower", braces(p.pad_lower),
           "--padding-upper", braces(p.pad_upper),
           "--in-dilation", braces(p.in_dilation),
           "--kernel-padding-lower", braces(p.k_pad_lower),
           "--kernel-padding-upper", braces(p.k_pad_upper),
           "--kernel-dilation", braces(p.k_dilation),
           "--single-phase", "all",
           "--convolution-options",
           '{"partialsType":"%s"}' % p.partials_type]
    if p.data_type == "quarter":
        cmd += ["--input-type", "quarter", "--output-type", "half"]
    else:
        cmd += ["--data-type", p.data_type]
    return cmd


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--seed", type=int, required=True)
    ap.add_argument("--input-type", default="all",
                    choices=["all", "half", "float", "quarter"])
    ap.add_argument("--max-flops", type=int, default=20_000_000)
    ap.add_argument("--max-elems", type=int, default=4_000_000)
    ap.add_argument("--binary",
                    default=os.path.join(HERE, "single_conv_layer"))
    ap.add_argument("--dry-run", action="store_true",
                    help="print the command, do not run it")
    args = ap.parse_args()
    rng = random.Random(args.seed)
    p = make_constrained_params(rng, args.input_type, args.max_flops,
                                args.max_elems)
    cmd = command(p, args.binary)
    print(" ".join(cmd), flush=True)
    if args.dry_run:
        return 0
    return subprocess.call(cmd)


if __name__ == "__main__":
    sys.exit(main())

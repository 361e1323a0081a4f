"""Pins the CPU oracle (oracle/conv_oracle.c) without running reference code:
library special cases, textbook identities, an independent index-definition
implementation, and slicing invariants.  A dropped term, wrong sign, transposed
operand or off-by-one in any transform fails at least one of these."""
import random

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import poplibs_amd as pa
from helpers import (conv_by_index_definition, make_params, output_size_def,
                     random_data, random_params)


def _torch_conv(p, acts, weights, biases):
    n = len(p.inputFieldShape)
    fn = {1: F.conv1d, 2: F.conv2d, 3: F.conv3d}[n]
    G, Co, Ci = (p.numConvGroups, p.outputChannelsPerConvGroup,
                 p.inputChannelsPerConvGroup)
    x = torch.from_numpy(acts)
    # asymmetric padding: pad explicitly (F.pad order: last dim first)
    pads = []
    for d in reversed(range(n)):
        pads += [p.inputTransform.paddingLower[d],
                 p.inputTransform.paddingUpper[d]]
    x = F.pad(x, pads)
    w = torch.from_numpy(weights).reshape(G * Co, Ci, *p.kernelShape)
    y = fn(x, w, torch.from_numpy(biases), stride=p.outputTransform.stride,
           dilation=p.kernelTransform.dilation, groups=G)
    return y.numpy()


CASES_TORCH = [
    dict(field=(8, 8), kernel=(3, 3), ci=3, co=4, pad=1),
    dict(field=(9, 7), kernel=(3, 2), ci=2, co=3, groups=2, stride=(2, 1),
         padLower=(1, 0), padUpper=(0, 2)),
    dict(field=(11,), kernel=(4,), ci=3, co=2, batch=3, stride=3, kdil=2,
         pad=3),
    dict(field=(5, 6, 4), kernel=(2, 3, 2), ci=2, co=2, groups=3, pad=(1, 0, 1),
         stride=(1, 2, 1), kdil=(2, 1, 1)),
    dict(field=(12, 12), kernel=(3, 3), groups=6, stride=2, pad=1, batch=2),
    dict(field=(6, 6), kernel=(1, 1), ci=5, co=7, batch=2),
    # benchmark config 1 shape class (N1 32x32 16->16 3x3 p1), reduced field
    dict(field=(16, 16), kernel=(3, 3), ci=16, co=16, pad=1),
]


@pytest.mark.parametrize("kw", CASES_TORCH)
def test_oracle_matches_torch_float64(oracle, kw):
    p = make_params(**kw)
    acts, weights, biases = random_data(p, seed=1)
    got = oracle.convolution(p, acts, weights, biases)
    want = _torch_conv(p, acts, weights, biases)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_oracle_1x1_is_matrix_product(oracle):
    p = make_params(field=(5, 3), kernel=(1, 1), ci=6, co=4, batch=2)
    acts, weights, _ = random_data(p, seed=2)
    got = oracle.convolution(p, acts, weights)
    want = np.einsum("bihw,oi->bohw", acts, weights[0, :, :, 0, 0])
    np.testing.assert_allclose(got, want, rtol=1e-13, atol=1e-13)


def test_oracle_delta_kernel_is_shifted_copy(oracle):
    # kernel with a single one at (0, 2): out[y][x] = in[y][x+2] (cross-
    # correlation, no kernel flip: lib/poplibs_test/Convolution.cpp:423-433)
    p = make_params(field=(4, 6), kernel=(2, 3))
    acts, _, _ = random_data(p, seed=3)
    weights = np.zeros((1, 1, 1, 2, 3))
    weights[0, 0, 0, 0, 2] = 1.0
    got = oracle.convolution(p, acts, weights)
    np.testing.assert_array_equal(got[0, 0], acts[0, 0, 0:3, 2:6])


def test_oracle_all_ones_box_sum_counts_border(oracle):
    p = make_params(field=(5, 5), kernel=(3, 3), pad=1)
    acts = np.ones((1, 1, 5, 5))
    weights = np.ones((1, 1, 1, 3, 3))
    got = oracle.convolution(p, acts, weights)[0, 0]
    counts = np.array([2, 3, 3, 3, 2])
    np.testing.assert_array_equal(got, np.outer(counts, counts))


def test_oracle_linearity_and_group_independence(oracle):
    p = make_params(field=(6, 5), kernel=(3, 2), ci=2, co=3, groups=2, pad=1,
                    stride=(2, 1))
    a1, w, _ = random_data(p, seed=4)
    a2, _, _ = random_data(p, seed=5)
    y1 = oracle.convolution(p, a1, w)
    y2 = oracle.convolution(p, a2, w)
    y12 = oracle.convolution(p, 2.0 * a1 - 3.0 * a2, w)
    np.testing.assert_allclose(y12, 2.0 * y1 - 3.0 * y2, rtol=1e-12,
                               atol=1e-12)
    # changing group 1's input leaves group 0's output untouched
    a3 = a1.copy()
    a3[:, 2:] += 1.0
    y3 = oracle.convolution(p, a3, w)
    np.testing.assert_array_equal(y3[:, :3], y1[:, :3])
    assert np.abs(y3[:, 3:] - y1[:, 3:]).max() > 0


def test_oracle_pm1_data_gives_exact_integers(oracle):
    # the harness's zero-tolerance mode (tools/single_conv_layer.cpp:979-1005)
    p = make_params(field=(7, 7), kernel=(3, 3), ci=4, co=3, pad=1)
    acts, weights, biases = random_data(p, seed=6, dist="pm1")
    got = oracle.convolution(p, acts, weights, biases)
    assert np.array_equal(got, np.round(got))
    want = _torch_conv(p, acts, weights, biases)
    np.testing.assert_array_equal(got, want)


def test_oracle_bias_is_added_to_output_padding_too(oracle):
    # lib/poplibs_test/Convolution.cpp:565-574
    p = make_params(field=(3,), kernel=(2,), opl=2, opu=1)
    acts, weights, _ = random_data(p, seed=7)
    got = oracle.convolution(p, acts, weights, np.array([5.0]))
    assert got.shape == (1, 1, 5)
    assert got[0, 0, 0] == 5.0 and got[0, 0, 1] == 5.0 and got[0, 0, 4] == 5.0
    inner = [acts[0, 0, i] * weights[0, 0, 0, 0]
             + acts[0, 0, i + 1] * weights[0, 0, 0, 1] + 5.0 for i in range(2)]
    np.testing.assert_allclose(got[0, 0, 2:4], inner, rtol=1e-14)


def test_oracle_known_small_answers(oracle):
    # hand-computed: in = [1,2,3,4], k = [1,10], input dilation 2 ->
    # dilated [1,0,2,0,3,0,4], conv out[i] = d[i] + 10 d[i+1]
    p = make_params(field=(4,), kernel=(2,), idil=2)
    got = oracle.convolution(p, np.array([[[1., 2, 3, 4]]]),
                             np.array([[[[1., 10]]]]))
    np.testing.assert_array_equal(got[0, 0], [1, 20, 2, 30, 3, 40])
    # flip input: reversed dilated array
    p = make_params(field=(4,), kernel=(2,), flipIn=True)
    got = oracle.convolution(p, np.array([[[1., 2, 3, 4]]]),
                             np.array([[[[1., 10]]]]))
    np.testing.assert_array_equal(got[0, 0], [34, 23, 12])
    # flip kernel -> true convolution
    p = make_params(field=(4,), kernel=(2,), flipK=True)
    got = oracle.convolution(p, np.array([[[1., 2, 3, 4]]]),
                             np.array([[[[1., 10]]]]))
    np.testing.assert_array_equal(got[0, 0], [12, 23, 34])
    # output truncation lower 1, stride 2: conv = [21,32,43] -> [32]
    p = make_params(field=(4,), kernel=(2,), otl=1, stride=2)
    got = oracle.convolution(p, np.array([[[1., 2, 3, 4]]]),
                             np.array([[[[1., 10]]]]))
    np.testing.assert_array_equal(got[0, 0], [32])
    # kernel padding lower 1: padded kernel [0,1,10] over [1,2,3,4]
    p = make_params(field=(4,), kernel=(2,), kpl=1)
    got = oracle.convolution(p, np.array([[[1., 2, 3, 4]]]),
                             np.array([[[[1., 10]]]]))
    np.testing.assert_array_equal(got[0, 0], [32, 43])
    # input truncation upper 1 + padding upper 2
    p = make_params(field=(4,), kernel=(2,), itu=1, padUpper=2)
    got = oracle.convolution(p, np.array([[[1., 2, 3, 4]]]),
                             np.array([[[[1., 10]]]]))
    np.testing.assert_array_equal(got[0, 0], [21, 32, 3, 0])


@pytest.mark.parametrize("seed", range(60))
def test_oracle_matches_index_definition_fuzz(oracle, seed):
    """Generalised transforms: array-staging oracle == closed-form index
    definition (two independent statements of the semantics)."""
    rng = random.Random(seed)
    p = random_params(rng, max_dims=3, max_field=6)
    acts, weights, biases = random_data(p, seed=seed)
    got = oracle.convolution(p, acts, weights, biases)
    want = conv_by_index_definition(p, acts, weights, biases)
    assert list(got.shape[2:]) == [output_size_def(p, d)
                                   for d in range(len(p.inputFieldShape))]
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_oracle_threads_do_not_change_bits(oracle):
    p = make_params(field=(9, 9), kernel=(3, 3), ci=5, co=6, groups=2, batch=3,
                    pad=1)
    acts, weights, biases = random_data(p, seed=8, dist="normal")
    a = oracle.convolution(p, acts, weights, biases, threads=1)
    b = oracle.convolution(p, acts, weights, biases, threads=4)
    assert np.array_equal(a, b)


def test_oracle_in_channel_split_sums_to_full(oracle):
    """Reduction of partials over an input-channel split
    (lib/poplin/Convolution.cpp:2762-2801) reproduces the full result."""
    p = make_params(field=(6, 6), kernel=(3, 3), ci=6, co=4, pad=1)
    acts, weights, _ = random_data(p, seed=9)
    full = oracle.convolution(p, acts, weights)
    h = make_params(field=(6, 6), kernel=(3, 3), ci=3, co=4, pad=1)
    part = (oracle.convolution(h, acts[:, :3], weights[:, :, :3])
            + oracle.convolution(h, acts[:, 3:], weights[:, :, 3:]))
    np.testing.assert_allclose(part, full, rtol=1e-13, atol=1e-13)


def test_oracle_output_slice_is_sub_convolution(oracle):
    """A tile of output rows is the convolution of the matching input rows
    with the tile range expressed as output truncation
    (getSubConvolution, lib/poplin/Convolution.cpp:357-494)."""
    p = make_params(field=(10, 5), kernel=(3, 3), ci=2, co=2, pad=1)
    acts, weights, _ = random_data(p, seed=10)
    full = oracle.convolution(p, acts, weights)
    # rows 4..7 of the 10 output rows: truncate output lower 4, upper 3
    sub = make_params(field=(10, 5), kernel=(3, 3), ci=2, co=2, pad=1,
                      otl=(4, 0), otu=(3, 0))
    np.testing.assert_array_equal(oracle.convolution(sub, acts, weights),
                                  full[:, :, 4:7])
    # and with the unused input rows sliced away (rows 3..7 feed outputs 4..6)
    sub2 = make_params(field=(5, 5), kernel=(3, 3), ci=2, co=2,
                       padLower=(0, 1), padUpper=(0, 1))
    np.testing.assert_array_equal(
        oracle.convolution(sub2, acts[:, :, 3:8], weights), full[:, :, 4:7])


def test_oracle_fp8_codec_tables(oracle):
    """Exhaustive decode table against the format definition, and encode as
    nearest-even inverse of decode (brute force over a dense grid)."""
    for fmt, mant, bias, maxv in ((oracle.E4M3, 3, 7, 448.0),
                                  (oracle.E5M2, 2, 15, 57344.0)):
        table = oracle.fp8_decode_table(fmt)
        for code in range(256):
            s = -1.0 if code & 0x80 else 1.0
            e = (code & 0x7f) >> mant
            m = code & ((1 << mant) - 1)
            if fmt == oracle.E4M3 and (code & 0x7f) == 0x7f:
                assert np.isnan(table[code])
                continue
            if fmt == oracle.E5M2 and e == 31:
                assert np.isinf(table[code]) if m == 0 else np.isnan(table[code])
                continue
            if e == 0:
                want = s * m * 2.0 ** (1 - bias - mant)
            else:
                want = s * (1 + m / 2.0 ** mant) * 2.0 ** (e - bias)
            assert table[code] == want
        finite = np.array(sorted(v for v in table if np.isfinite(v)))
        assert finite.max() == maxv
        # every representable value round-trips
        for code in range(256):
            if np.isfinite(table[code]):
                got = int(oracle.fp8_encode([table[code]], fmt)[0])
                assert table[got] == table[code]
        # brute-force nearest-even on a grid of in-range values
        g = np.random.default_rng(0)
        xs = np.concatenate([g.uniform(-maxv, maxv, 3000),
                             g.normal(0, 1, 3000), g.normal(0, 0.01, 2000)])
        pos = finite[finite >= 0]
        codes = oracle.fp8_encode(xs, fmt)
        for x, c in zip(xs, codes):
            a = abs(x)
            j = np.searchsorted(pos, a)
            lo = pos[max(j - 1, 0)]
            hi = pos[min(j, len(pos) - 1)]
            if a - lo < hi - a:
                want = lo
            elif a - lo > hi - a:
                want = hi
            else:  # tie -> even mantissa code
                clo = int(oracle.fp8_encode([lo], fmt)[0])
                want = lo if (clo & 1) == 0 else hi
            assert abs(table[c]) == want, (x, c, want)
            assert (c >> 7) == (1 if x < 0 else 0) or want == 0
        # saturation and metadata scaling
        assert table[int(oracle.fp8_encode([1e9], fmt)[0])] == maxv
        assert table[int(oracle.fp8_encode([-1e9], fmt)[0])] == -maxv
    md = oracle.quarter_metadata(oracle.E4M3, -3)
    assert md == (0x80 | (0x3f & -3))
    vals = oracle.quarter_to_double(np.array([0x38, 0xb8], dtype=np.uint8), md)
    np.testing.assert_array_equal(vals, [0.125, -0.125])

"""Host-side descriptor algebra (ConvParams, ConvUtil, MAC counting, options,
planner) exercised through the C ABI; no GPU needed.  Known answers come from
the reference's own unit tests (cited), the rest is pinned by brute force
against an independent Python statement of the index definition."""
import os
import random

import numpy as np
import pytest

import poplibs_amd as pa
from poplibs_amd import MxconvError, Status, capi
from helpers import (NONE, input_index_def, make_params, output_size_def,
                     random_data, random_params)

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---- known answers held by the reference's tests --------------------------

def test_getInputRange_flip_acts_and_weights():
    # tests/poplin/ConvUtilTest.cpp:14-32
    p = pa.ConvParams(pa.FLOAT, None, 1, [3, 1], [5, 1], 1, 1, 1)
    p.inputTransform.paddingLower = [2, 0]
    p.inputTransform.paddingUpper = [2, 0]
    p.inputTransform.flip = [True, False]
    p.kernelTransform.flip = [True, False]
    assert p.getInputRange(0, (0, 2), 1) == (0, 2)


def test_getKernelRange_truncate_input():
    # tests/poplin/ConvUtilTest.cpp:34-51
    p = pa.ConvParams(pa.FLOAT, None, 1, [3], [4], 1, 1, 1)
    p.inputTransform.truncationUpper = [1]
    p.inputTransform.dilation = [2]
    p.inputTransform.paddingLower = [1]
    assert p.getKernelRange(0, (0, 1), (0, 3)) == (1, 4)


def test_read_conv_params_from_json():
    # tests/poplin/ConvTest.cpp:651-682
    uut = pa.ConvParams.from_json("""
    {
      "dataType": "float",
      "batchSize": 1,
      "numConvGroups": 2,
      "inputChannelsPerConvGroup": 3,
      "outputChannelsPerConvGroup": 4,
      "kernelShape": [50, 60],
      "inputFieldShape": [70, 80],
      "inputTransform": {
        "truncationLower": [1, 2],
        "paddingUpper": [3, 4],
        "flip": [true, false]
      },
      "outputTransform": {
        "stride": [5, 6]
      }
    }""")
    expected = pa.ConvParams(pa.FLOAT, None, 1, [70, 80], [50, 60], 3, 4, 2)
    expected.inputTransform.truncationLower = [1, 2]
    expected.inputTransform.paddingUpper = [3, 4]
    expected.inputTransform.flip = [True, False]
    expected.outputTransform.stride = [5, 6]
    assert uut == expected
    assert uut.compare(expected) == 0 and uut.hash() == expected.hash()


def test_json_fixtures_of_the_reference():
    dw = pa.ConvParams.from_json(
        open(os.path.join(GOLDEN, "depthwise_conv_half.json")).read())
    assert dw == pa.ConvParams(pa.HALF, None, 1, [28, 28], [5, 5], 1, 1, 24)
    pw = pa.ConvParams.from_json(
        open(os.path.join(GOLDEN, "pointwise_conv_float.json")).read())
    assert pw == pa.ConvParams(pa.FLOAT, None, 2, [17, 32], [1, 1], 16, 25, 1)
    assert pw.getOutputFieldShape() == [17, 32]


def test_json_input_output_types_and_errors():
    p = pa.ConvParams.from_json(
        '{"inputType": "quarter", "outputType": "half", "batchSize": 2,'
        ' "numConvGroups": 1, "inputChannelsPerConvGroup": 16,'
        ' "outputChannelsPerConvGroup": 8, "inputFieldShape": [4],'
        ' "kernelShape": [1], "kernelTransform": {"dilation": [3]}}')
    assert (p.inputType, p.outputType) == (pa.QUARTER, pa.HALF)
    assert p.kernelTransform.dilation == [3]
    with pytest.raises(MxconvError) as e:  # lib/poplin/ConvParams.cpp:417-420
        pa.ConvParams.from_json('{"inputFieldShape": [4, 4], "kernelShape": [1]}')
    assert e.value.status == Status.INVALID_PARAMS
    with pytest.raises(MxconvError):
        pa.ConvParams.from_json('{"dataType": "double"}')
    with pytest.raises(MxconvError):
        pa.ConvParams.from_json('{"batchSize": ')


def test_validate_options():
    # tests/poplin/ConvTest.cpp:684-698
    pa.validate_options({"partialsType": "half"})
    for bad in ({"partialsType": "invalid_value"}, {"invalid_key": "half"}):
        with pytest.raises(MxconvError) as e:
            pa.validate_options(bad)
        assert e.value.status == Status.INVALID_OPTION
    pa.validate_options({"pass": "TRAINING_FWD",
                         "availableMemoryProportion": "0.4",
                         "enableFastReduce": "true"})
    for bad in ({"pass": "FWD"}, {"availableMemoryProportion": "-1"},
                {"enableFastReduce": "maybe"}):
        with pytest.raises(MxconvError):
            pa.validate_options(bad)


def _pc(text):
    pa.validate_options({"planConstraints": text})


def _pc_bad(text):
    with pytest.raises(MxconvError) as e:
        _pc(text)
    assert e.value.status == Status.INVALID_OPTION


def test_plan_constraints_structure():
    # tests/poplin/ConvOptionsTest.cpp:12-107 restated on the JSON form
    _pc('{}')
    _pc('{"0": {}}')
    _pc('{"0": {}, "2": {}, " 5": {}}')
    _pc_bad('{"": {}}')
    _pc_bad('{"-1": {}}')
    _pc_bad('{"a watched pot never boils": {}}')
    _pc_bad('0')
    # partition variables per dimension
    _pc('{"0": {"partition": {"fieldSplit": {"0": 4, "2": 5}}}}')
    _pc_bad('{"0": {"partition": {"fieldSplit": '
            '{"5": "a watched pot never boils"}}}}')
    _pc_bad('{"0": {"partition": {"fieldSplit": 0}}}')
    _pc_bad('{"0": {"partition": {"fieldSplit": {"hello": "world"}}}}')
    # split variables
    _pc('{"0": {"partition": {"inChanSplit": {"serial": 4, "parallel": 5}}}}')
    _pc_bad('{"0": {"partition": {"inChanSplit": '
            '{"serial": "a watched pot never boils"}}}}')
    _pc_bad('{"0": {"partition": {"outChanSplit": {"hello": "world"}}}}')
    # transform
    _pc('{"0": {"transform": {"swapOperands": false}}}')
    _pc_bad('{"0": {"transform": {"a watched pot never boils": {}}}}')
    _pc_bad('{"0": {"transform": {"swapOperands": '
            '"a watched pot never boils"}}}')
    _pc_bad('{"0": {"transform": 0}}')
    # partition scalars
    _pc('{"0": {"partition": {"convGroupSplit": 4}}}')
    _pc_bad('{"0": {"partition": {"a watched pot never boils": {}}}}')
    _pc_bad('{"0": {"partition": {"convGroupSplit": '
            '"a watched pot never boils"}}}')
    _pc_bad('{"0": {"something": {}}}')
    # method (lib/poplin/ConvOptions.cpp:275-299)
    for m in ("AMP", "SLIC", "HMAC", "VMAC", "OUTER_PRODUCT"):
        _pc('{"method": {"type": "%s"}}' % m)
    _pc_bad('{"method": {"type": "WINOGRAD"}}')
    # the complete constraint of tests/poplin/ConvPlanTest.cpp:155-175
    _pc('''{"method": {"type": "HMAC"}, "inChansPerGroup": 1,
            "partialChansPerGroup": 1,
            "0": {"transform": {"swapOperands": false, "expandDims": [],
                                "outChanFlattenDims": []},
                  "partition": {"fieldSplit": {"0": 1, "1": 1},
                                "batchSplit": 1,
                                "outChanSplit": {"parallel": 1, "serial": 1},
                                "kernelSplit": {"0": 1, "1": 1},
                                "inChanSplit": {"parallel": 1, "serial": 1},
                                "convGroupSplit": 1}}}''')


# ---- validate (lib/poplin/ConvParams.cpp:172-266) -------------------------

@pytest.mark.parametrize("mutate,fragment", [
    (lambda p: p.kernelShape.append(1), "kernel field dimensions"),
    (lambda p: p.outputTransform.stride.__setitem__(0, 0), "Stride"),
    (lambda p: p.inputTransform.dilation.__setitem__(1, 0), "Input dilation"),
    (lambda p: p.kernelTransform.dilation.__setitem__(0, 0),
     "Kernel dilation"),
    (lambda p: p.inputTransform.paddingLower.append(0), "dimensions"),
    (lambda p: p.inputTransform.truncationLower.__setitem__(0, 9),
     "more than the size of the field"),
    (lambda p: p.kernelTransform.truncationUpper.__setitem__(1, 4),
     "more than the size of the kernel"),
    (lambda p: (p.kernelTransform.truncationLower.__setitem__(0, 3)),
     "zero size"),
    (lambda p: p.kernelTransform.dilation.__setitem__(0, 5),
     "less than the transformed kernel"),
    (lambda p: p.outputTransform.truncationLower.__setitem__(0, 7),
     "Output truncation"),
])
def test_validate_rejects(mutate, fragment):
    p = make_params(field=(8, 8), kernel=(3, 3))
    p.validate()
    mutate(p)
    with pytest.raises(MxconvError) as e:
        p.validate()
    assert e.value.status == Status.INVALID_PARAMS
    assert fragment in e.value.message, e.value.message


# ---- sizes: closed forms (lib/poplin/ConvParams.cpp:631-698) --------------

def test_baseline_config_sizes_and_flops():
    c1 = make_params(pa.FLOAT, field=(32, 32), kernel=(3, 3), ci=16, co=16,
                     pad=1)
    c2 = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                     co=128, pad=1)
    c3 = make_params(pa.HALF, batch=32, field=(56, 56), kernel=(1, 1), ci=256,
                     co=64)
    c4 = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                     groups=96, stride=2, pad=1)
    c5 = make_params(pa.QUARTER, pa.HALF, batch=64, field=(14, 14),
                     kernel=(3, 3), ci=256, co=256, pad=1)
    assert [c.getOutputFieldShape() for c in (c1, c2, c3, c4, c5)] == [
        [32, 32], [28, 28], [56, 56], [56, 56], [14, 14]]
    assert [c.getFwdFlops() for c in (c1, c2, c3, c4, c5)] == [
        4524032, 7050625024, 3288334336, 171350016, 13421772800]
    # closed form for 3x3 pad 1 on HxW: sum over taps of valid outputs
    assert c2.getNumberOfMACs() == 32 * 128 * 128 * (28 + 27 + 27) ** 2
    # c4: stride 2 over 112 with pad 1: rows k=0 -> 55 outputs, k=1,2 -> 56
    assert c4.getNumberOfMACs() == 32 * 96 * (55 + 56 + 56) ** 2


@pytest.mark.parametrize("seed", range(40))
def test_sizes_match_definition_fuzz(seed):
    p = random_params(random.Random(seed), max_dims=4, max_field=9)
    for d in range(p.getNumFieldDims()):
        assert p.getOutputSize(d) == output_size_def(p, d)
        it = p.inputTransform
        trunc = p.inputFieldShape[d] - it.truncationLower[d] \
            - it.truncationUpper[d]
        assert p.getTruncatedInputSize(d) == trunc
        dil = 0 if trunc == 0 else 1 + (trunc - 1) * it.dilation[d]
        assert p.getTransformedInputSize(d) == \
            it.paddingLower[d] + dil + it.paddingUpper[d]
        assert p.getUntransformedOutputSize(d) == \
            p.getTransformedInputSize(d) - p.getTransformedKernelSize(d) + 1


# ---- index and range algebra against brute force --------------------------

@pytest.mark.parametrize("seed", range(40))
def test_index_and_ranges_match_brute_force(seed):
    rng = random.Random(100 + seed)
    p = random_params(rng, max_dims=2, max_field=8)
    for d in range(p.getNumFieldDims()):
        O, K, I = p.getOutputSize(d), p.kernelShape[d], p.inputFieldShape[d]
        table = {}
        for o in range(O):
            for k in range(K):
                want = input_index_def(p, d, o, k)
                got = p.getInputIndex(d, o, k)
                assert got == (NONE if want is None else want)
                if want is not None:
                    table[(o, k)] = want
                    assert p.getKernelIndex(d, o, want) == k
        for o in range(O):
            for i in range(I):
                ks = [k for k in range(K) if table.get((o, k)) == i]
                got = p.getKernelIndex(d, o, i)
                assert got == (ks[0] if ks else NONE)

        def span(values):
            values = list(values)
            return (min(values), max(values) + 1) if values else (0, 0)

        for _ in range(6):
            o0 = rng.randint(0, O)
            o1 = rng.randint(o0, O)
            k0 = rng.randint(0, K)
            k1 = rng.randint(k0, K)
            i0 = rng.randint(0, I)
            i1 = rng.randint(i0, I)
            pairs = [(o, k, i) for (o, k), i in table.items()
                     if o0 <= o < o1]
            assert p.getOutputRangeForKernelRange(d, (o0, o1), (k0, k1)) == \
                span(o for o, k, i in pairs if k0 <= k < k1)
            assert p.getOutputRangeForInputRange(d, (o0, o1), (i0, i1)) == \
                span(o for o, k, i in pairs if i0 <= i < i1)
            assert p.getInputRange(d, (o0, o1), (k0, k1)) == \
                span(i for o, k, i in pairs if k0 <= k < k1)
            assert p.getKernelRange(d, (o0, o1), (i0, i1)) == \
                span(k for o, k, i in pairs if i0 <= i < i1)


@pytest.mark.parametrize("seed", range(40))
def test_number_of_macs_counts_index_pairs(seed):
    """getNumberOfMACs == number of (o, k) pairs per dimension with an input
    element, times channels (lib/poplin/PerformanceEstimation.hpp:1641-1666).
    The reference's formula divides a range size by a stride, which equals the
    pair count whenever the participating outputs of a kernel index are
    evenly spaced - true for every parameter set."""
    p = random_params(random.Random(200 + seed), max_dims=3, max_field=9)
    want = (p.numConvGroups * p.batchSize * p.outputChannelsPerConvGroup
            * p.inputChannelsPerConvGroup)
    for d in range(p.getNumFieldDims()):
        want *= sum(input_index_def(p, d, o, k) is not None
                    for o in range(p.getOutputSize(d))
                    for k in range(p.kernelShape[d]))
    assert p.getNumberOfMACs() == want
    assert p.getFwdFlops() == 2 * want


# ---- canonicalize (lib/poplin/ConvParams.cpp:468-629) ---------------------

@pytest.mark.parametrize("seed", range(50))
def test_canonicalize_invariants(oracle, seed):
    p = random_params(random.Random(300 + seed), max_dims=3, max_field=7)
    c = p.canonicalize()
    c.validate()
    # shapes preserved (lib/poplin/ConvParams.cpp:626), idempotent
    # (lib/poplin/CanonicalConvParams.hpp:15-19)
    assert c.getOutputFieldShape() == p.getOutputFieldShape()
    assert (c.inputFieldShape, c.kernelShape) == (p.inputFieldShape,
                                                  p.kernelShape)
    assert c.canonicalize() == c
    # and it is the same function of the data
    acts, weights, biases = random_data(p, seed)
    np.testing.assert_array_equal(
        oracle.convolution(c, acts, weights, biases),
        oracle.convolution(p, acts, weights, biases))
    assert c.getNumberOfMACs() == p.getNumberOfMACs()


def test_canonicalize_known_forms():
    # config 4: the upper padding row/column is never read
    c4 = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                     groups=96, stride=2, pad=1).canonicalize()
    assert c4.inputTransform.paddingLower == [1, 1]
    assert c4.inputTransform.paddingUpper == [0, 0]
    assert c4.outputTransform.stride == [2, 2]
    # one output element: stride collapses to 1
    p = make_params(field=(5,), kernel=(5,), stride=3).canonicalize()
    assert p.outputTransform.stride == [1]
    # flip of a single surviving element is dropped, paddings swap
    p = make_params(field=(4,), kernel=(1,), itl=1, itu=2, flipIn=True,
                    padLower=2, padUpper=0, idil=3).canonicalize()
    assert p.inputTransform.flip == [False]
    assert p.inputTransform.dilation == [1]
    # all-zero output -> the zero convolution of getZeroConv
    z = make_params(field=(2,), kernel=(1,), padLower=4, otu=4)
    assert z.isZeroConvolution()
    zc = z.canonicalize()
    assert zc.inputTransform.truncationUpper == [2]
    assert zc.kernelTransform.truncationUpper == [1]
    assert zc.outputTransform.paddingUpper == zc.getOutputFieldShape()
    assert not make_params(field=(4,), kernel=(2,)).isZeroConvolution()
    assert make_params(field=(4,), kernel=(2,), ci=0).isZeroConvolution()


# ---- ordering, hashing, printing ------------------------------------------

def test_compare_hash_and_print():
    a = make_params(field=(4, 4), kernel=(3, 3), pad=1)
    b = make_params(field=(4, 4), kernel=(3, 3), pad=1)
    c = make_params(field=(4, 4), kernel=(3, 3), pad=1, stride=2)
    assert a.compare(b) == 0 and a.hash() == b.hash()
    assert a.compare(c) != 0 and a.compare(c) == -c.compare(a)
    assert a.hash() != c.hash()
    text = str(c)
    # fixed layout of lib/poplin/ConvParams.cpp:292-363
    assert text.startswith("\n  Params:\n        inputType                  "
                           "float\n")
    assert "        stride                     {2,2}\n" in text
    assert "        flipInput                  {0,0}\n" in text
    assert text.endswith("        outputFieldShape           {2,2}\n")


# ---- planner --------------------------------------------------------------

def _kernel_of(p, options=None):
    text = pa.Plan(p, options).describe()
    for name in ("implicit GEMM", "depthwise direct", "generic direct"):
        if name in text:
            return name
    raise AssertionError(text)


def test_planner_choices():
    c1 = make_params(pa.FLOAT, field=(32, 32), kernel=(3, 3), ci=16, co=16,
                     pad=1)
    c2 = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                     co=128, pad=1)
    c4 = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                     groups=96, stride=2, pad=1)
    c5 = make_params(pa.QUARTER, pa.HALF, batch=64, field=(14, 14),
                     kernel=(3, 3), ci=256, co=256, pad=1)
    assert _kernel_of(c1) == "implicit GEMM"       # fp32 MFMA
    assert _kernel_of(c2) == "implicit GEMM"
    assert _kernel_of(c4) == "depthwise direct"
    assert _kernel_of(c5) == "implicit GEMM"
    # a dilated input (what the backward pass of a strided layer brings) and
    # a kernel of many taps (what a weight update pass brings) stay on the
    # matrix cores, with other ways of telling which taps read the input
    dilated = pa.Plan(make_params(pa.HALF, field=(8, 8), kernel=(3, 3), ci=8,
                                  co=8, idil=2)).describe()
    assert "implicit GEMM" in dilated and "4 phases" in dilated
    # ... with a window that moves by more than one pixel over the stuffed
    # input there are no such phases: every tap's position is worked out
    strided = pa.Plan(make_params(pa.HALF, field=(8, 8), kernel=(3, 3), ci=8,
                                  co=8, idil=2, stride=2)).describe()
    assert "implicit GEMM" in strided and "arithmetic" in strided
    many = pa.Plan(make_params(pa.HALF, batch=128, field=(28, 28),
                               kernel=(28, 28), ci=32, co=128, pad=1))
    assert "implicit GEMM" in many.describe()
    assert "ranges of valid kernel rows" in many.describe()
    # few output tiles, long K: K is cut into parts, over narrow tiles
    assert "K split into parts         14" in many.describe()
    assert "block M x N x K            128 x 64 x 64" in many.describe()
    assert many.buffer_bytes(4) == 14 * 128 * 9 * 128 * 4
    assert "K split" not in pa.Plan(c2).describe()
    # ... unless the parts' round trip through memory costs more than it
    # saves: 98 tiles of 16 k-steps stay whole
    assert "K split" not in pa.Plan(make_params(
        pa.HALF, batch=32, field=(14, 14), kernel=(1, 1), ci=1024,
        co=256)).describe()
    # (two parts over 104 narrow tiles rather than four over 52 wide ones)
    assert "K split into parts         2" in pa.Plan(make_params(
        pa.HALF, batch=32, field=(7, 7), kernel=(3, 3), ci=512, co=512,
        pad=1)).describe()
    # one workgroup per CU or fewer: four LDS stages; more workgroups than
    # CUs: two stages, two workgroups per CU
    # (c2 itself goes to the kernel with the input patch resident in LDS)
    streaming = {"planConstraints": '{"gfx950": {"patch": 0}}'}
    assert "LDS stages                 4" in pa.Plan(c2, streaming).describe()
    assert "input rows of the tile resident" in pa.Plan(c2).describe()
    c2_large = make_params(pa.HALF, batch=256, field=(28, 28), kernel=(3, 3),
                           ci=128, co=128, pad=1)
    assert "LDS stages                 2" in \
        pa.Plan(c2_large, streaming).describe()
    assert "MFMA blocks of 16 pixels" in pa.Plan(c2_large).describe()
    forced = pa.Plan(c2, {"planConstraints": '{"gfx950": {"stages": 2}}'})
    assert "LDS stages                 2" in forced.describe()
    with pytest.raises(MxconvError):
        pa.Plan(c2, {"planConstraints": '{"gfx950": {"stages": 3}}'})
    # transforms outside the fast subset fall back
    assert _kernel_of(make_params(pa.HALF, field=(8, 8), kernel=(3, 3), ci=8,
                                  co=8, flipIn=True)) == "generic direct"
    # (a flipped, truncated or padded kernel is the stored one with its taps
    # picked in another order: the weight packing's business)
    assert _kernel_of(make_params(pa.HALF, field=(8, 8), kernel=(3, 3), ci=8,
                                  co=8, flipK=True)) == "implicit GEMM"
    # three field dimensions: the matrix cores take undilated inputs; a
    # depth the window does not slide over is batch
    assert _kernel_of(make_params(pa.HALF, field=(8, 8, 8), kernel=(3, 3, 3),
                                  ci=8, co=8)) == "implicit GEMM"
    many3d = pa.Plan(make_params(pa.HALF, field=(8, 8, 8), kernel=(3, 3, 4),
                                 ci=8, co=8)).describe()
    assert "implicit GEMM" in many3d and "ranges of valid kernel" in many3d
    assert "2 phases" in pa.Plan(make_params(
        pa.HALF, field=(8, 8, 8), kernel=(3, 3, 3), ci=8, co=8,
        idil=(1, 2, 1))).describe()
    assert _kernel_of(make_params(pa.HALF, field=(8, 8, 8), kernel=(3, 3, 3),
                                  ci=8, co=8, idil=(1, 2, 1),
                                  stride=(1, 2, 1))) == "generic direct"
    assert _kernel_of(make_params(pa.HALF, field=(8, 8, 8), kernel=(3, 3, 3),
                                  ci=8, co=8, opu=(0, 1, 0))) == \
        "implicit GEMM"
    folded = pa.Plan(make_params(pa.HALF, batch=2, field=(5, 9, 9),
                                 kernel=(1, 7, 7), ci=8, co=8))
    assert "gemm M x N x K             90 x 8 x 392" in folded.describe()
    assert _kernel_of(make_params(pa.HALF, field=(4, 8, 8, 8),
                                  kernel=(1, 3, 3, 3), ci=8, co=8)) == \
        "generic direct"
    # channel counts that are no whole 16-byte vector are padded for the
    # matrix cores (a zero-filled copy in the workspace) ...
    few = pa.Plan(make_params(pa.HALF, batch=2, field=(32, 32), kernel=(3, 3),
                              ci=5, co=64))
    assert "implicit GEMM" in few.describe()
    assert "input channels padded      5 -> 8" in few.describe()
    assert few.buffer_bytes(4) == 2 * 32 * 32 * 8 * 2
    assert few.buffer_bytes(0) == 2 * 32 * 32 * 5 * 2   # the caller's input
    # ... unless there are at most 4 of them in one group: then a kernel
    # row's pixels, neighbours in a channels-last image, make one k-step, and
    # the input is read as it is
    thin = pa.Plan(make_params(pa.HALF, batch=2, field=(32, 32),
                               kernel=(3, 3), ci=3, co=64))
    assert "kernel rows as k-steps" in thin.describe()
    assert "a kernel row's 3 x 3 = 9 neighbouring elements" in thin.describe()
    # (two chunks of 8 per kernel row, six in all: two k-steps of four)
    assert "x 64 x 64 (" in thin.describe()
    assert thin.buffer_bytes(4) == 0
    assert thin.buffer_bytes(1) == 4 * 2 * 64 * 8 * 2
    off = {"planConstraints": '{"gfx950": {"thinInput": 0}}'}
    assert "input channels padded      3 -> 8" in pa.Plan(
        make_params(pa.HALF, batch=2, field=(32, 32), kernel=(3, 3), ci=3,
                    co=64), off).describe()
    # (48 output channels: three blocks of 16; 80: not this kernel's)
    assert "kernel rows as k-steps" in pa.Plan(make_params(
        pa.HALF, batch=2, field=(32, 32), kernel=(5, 5), ci=4,
        co=48)).describe()
    assert "kernel rows as k-steps" not in pa.Plan(make_params(
        pa.HALF, batch=2, field=(32, 32), kernel=(5, 5), ci=4,
        co=80)).describe()
    with pytest.raises(MxconvError, match="thinInput"):
        pa.Plan(make_params(pa.HALF, batch=2, field=(32, 32), kernel=(5, 5),
                            ci=4, co=80),
                {"planConstraints": '{"gfx950": {"thinInput": 1}}'})
    # ... except when there is too little work to pay for the copy
    assert _kernel_of(make_params(pa.HALF, field=(8, 8), kernel=(3, 3), ci=4,
                                  co=8)) == "generic direct"
    # method names of the reference steer the choice
    hmac = {"planConstraints": '{"method": {"type": "HMAC"}}'}
    assert _kernel_of(c2, hmac) == "generic direct"
    assert _kernel_of(c4, {"planConstraints":
                           '{"method": {"type": "AMP"}}'}) == "depthwise direct"
    forced = {"planConstraints": '{"gfx950": {"kernel": "generic"}}'}
    assert _kernel_of(c2, forced) == "generic direct"
    flipped = make_params(pa.HALF, field=(8, 8), kernel=(3, 3), ci=8, co=8,
                          flipIn=True)
    with pytest.raises(MxconvError) as e:
        pa.Plan(flipped, {"planConstraints": '{"gfx950": {"kernel": "igemm"}}'})
    assert e.value.status == Status.INVALID_OPTION
    with pytest.raises(MxconvError):
        pa.Plan(c2, {"planConstraints": '{"gfx950": {"blockM": 96}}'})


def test_plan_buffers_and_type_rules():
    from poplibs_amd import capi
    c2 = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                     co=128, pad=1)
    plan = pa.Plan(c2)
    assert plan.buffer_bytes(capi.BUF_INPUT) == 6422528
    assert plan.buffer_bytes(capi.BUF_WEIGHTS_EXTERNAL) == 294912
    assert plan.buffer_bytes(capi.BUF_OUTPUT) == 6422528
    assert plan.buffer_bytes(capi.BUF_BIAS) == 256
    # quarter input requires half output (lib/poplin/ConvValidation.cpp:55-61)
    bad = make_params(pa.QUARTER, pa.FLOAT, field=(4, 4), kernel=(1, 1), ci=16,
                      co=16)
    with pytest.raises(MxconvError) as e:
        pa.Plan(bad)
    assert e.value.status == Status.INVALID_PARAMS
    # invalid parameters are rejected at planning time
    with pytest.raises(MxconvError):
        pa.Plan(make_params(field=(2, 2), kernel=(3, 3)))
    # fwd on a quarter plan needs the metadata entry point; no GPU touched
    q = pa.Plan(make_params(pa.QUARTER, pa.HALF, field=(4, 4), kernel=(1, 1),
                            ci=16, co=16))
    with pytest.raises(MxconvError) as e:
        q.fwd(1, 1, 1)
    assert "mxconv_fwd_quarter" in e.value.message


def test_plan_estimated_costs():
    """mxconv_plan_estimated_costs (reportPlanEstimatedCosts,
    include/poplin/Convolution.hpp:590-611): the chosen tiling's estimate in
    cycles at 2.1 GHz, the workspace as temporary memory, unknown for the
    generic kernel."""
    import re
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    plan = pa.Plan(p)
    cycles, memory = plan.estimated_costs()
    chosen = re.search(r"^\s+\*.*?([\d.]+) us$", plan.describe(), re.M)
    assert abs(cycles - float(chosen.group(1)) * 2100) <= 2100 * 0.05 + 1
    assert memory == 0 == plan.buffer_bytes(capi.BUF_WORKSPACE)
    # streamed kernels: time grows with the bytes moved
    small = make_params(pa.HALF, batch=32, field=(112, 112), kernel=(3, 3),
                        groups=96, stride=2, pad=1)
    large = make_params(pa.HALF, batch=64, field=(112, 112), kernel=(3, 3),
                        groups=96, stride=2, pad=1)
    a, b = pa.Plan(small).estimated_costs()[0], \
        pa.Plan(large).estimated_costs()[0]
    assert 17.9 * 0.75 < a / 2100 < 17.9 * 1.25  # 17.9 us measured
    assert 1.7 * a < b < 2.0 * a  # one launch overhead, twice the bytes
    # K split: the fp32 partial tiles are temporary memory
    deep = pa.Plan(make_params(pa.HALF, batch=4, field=(14, 14),
                               kernel=(3, 3), ci=256, co=256, pad=1),
                   {"planConstraints": '{"gfx950": {"patch": 0}}'})
    assert "K split into parts" in deep.describe()
    cycles, memory = deep.estimated_costs()
    assert memory == deep.buffer_bytes(capi.BUF_WORKSPACE) > 0
    assert cycles != pa.Plan.COST_UNKNOWN
    # outside the cost model
    generic = pa.Plan(make_params(pa.FLOAT, pa.FLOAT, batch=1, field=(5, 5),
                                  kernel=(3, 3), ci=3, co=5))
    assert "generic direct" in generic.describe()
    assert generic.estimated_costs()[0] == pa.Plan.COST_UNKNOWN


def test_plan_detailed_costs():
    """mxconv_plan_detailed_costs (reportDetailedPlanEstimatedCosts,
    include/poplin/Convolution.hpp:613-676): the estimate by phase.  The
    phases add up to the total, the total is what
    mxconv_plan_estimated_costs returns, and each phase appears exactly where
    the plan has that step."""
    def parts(plan):
        d = plan.detailed_costs()
        assert d["total"] == plan.estimated_costs()
        assert sum(d[k][0] for k in ("rearrangement", "compute",
                                     "reduction")) == d["total"][0]
        assert d["rearrangement"][1] + d["reduction"][1] <= d["total"][1]
        assert d["parallelSplit"] >= 1 and d["serialSplit"] >= 1
        return d
    # one kernel and nothing else; 224 workgroups in one round
    d = parts(pa.Plan(make_params(pa.HALF, batch=32, field=(28, 28),
                                  kernel=(3, 3), ci=128, co=128, pad=1)))
    assert d["rearrangement"] == (0, 0) and d["reduction"] == (0, 0)
    assert (d["parallelSplit"], d["serialSplit"]) == (224, 1)
    # many tiles: rounds of them, no more side by side than the chip holds
    d = parts(pa.Plan(make_params(pa.HALF, batch=128, field=(56, 56),
                                  kernel=(3, 3), ci=64, co=64, pad=1)))
    assert d["serialSplit"] > 1 and d["parallelSplit"] in (256, 512)
    # K split over workgroups: the second kernel and its fp32 tiles
    deep = pa.Plan(make_params(pa.HALF, batch=4, field=(14, 14),
                               kernel=(3, 3), ci=256, co=256, pad=1),
                   {"planConstraints": '{"gfx950": {"patch": 0}}'})
    assert "K split into parts" in deep.describe()
    d = parts(deep)
    assert d["reduction"][1] == deep.buffer_bytes(capi.BUF_WORKSPACE) > 0
    # the second kernel (4.5 us) and the partial tiles out and in at 6.4 TB/s
    assert d["reduction"][0] == round(
        (4.5 + 2 * d["reduction"][1] / 6.4e6) * 2100)
    # six input channels: copied into whole vectors first
    stem = pa.Plan(make_params(pa.HALF, batch=8, field=(56, 56),
                               kernel=(3, 3), ci=6, co=64, pad=1))
    assert "generic direct" not in stem.describe()
    d = parts(stem)
    assert d["rearrangement"][0] > 2.0 * 2100  # at least a launch
    assert d["rearrangement"][1] == stem.buffer_bytes(capi.BUF_WORKSPACE) > 0
    assert d["compute"][0] > 0
    # the weight update pass of a dense layer on its own tensors: the matrix
    # core kernel, then the ordered sum of the chunks' tiles
    wu = pa.WeightUpdatePlan(make_params(pa.HALF, batch=32, field=(28, 28),
                                         kernel=(3, 3), ci=128, co=128,
                                         pad=1))
    d = parts(wu)
    assert d["reduction"][0] > 0 and d["reduction"][1] > 0
    assert d["compute"][0] > d["reduction"][0]
    # outside the cost model
    generic = pa.Plan(make_params(pa.FLOAT, pa.FLOAT, batch=1, field=(5, 5),
                                  kernel=(3, 3), ci=3, co=5))
    d = generic.detailed_costs()
    assert all(d[k][0] == pa.Plan.COST_UNKNOWN
               for k in ("rearrangement", "compute", "reduction", "total"))


def test_planner_weighs_tilings_and_reports_them():
    """The matrix-core plan lists the tilings it weighed with their estimated
    times, picks the cheapest, and says how many CUs the launch occupies;
    planConstraints force each of them (role of choosePlan,
    lib/poplin/ConvPlan.cpp:502-565, and of reportPlanEstimatedCosts)."""
    import json
    import re
    p = make_params(pa.HALF, batch=32, field=(28, 28), kernel=(3, 3), ci=128,
                    co=128, pad=1)
    text = pa.Plan(p).describe()
    # 25 088 pixels: 224 tiles of 112 (seven whole 16-pixel blocks; 256 equal
    # tiles of 98 cost each workgroup the same seven) rather than 196 of 128
    assert "224 on 256 CUs (224 busy, 1 round(s) of tiles)" in text
    assert "block M x N x K            112 x 128 x 64" in text
    rows = re.findall(r"^\s+(\*?)\s*(streaming|resident patch) (.*?)\s+(\d+)"
                      r"\s+(\d+)\s+([\d.]+)\s+(\d+)\s+([\d.]+) us$", text,
                      re.M)
    assert len(rows) == 4, text
    chosen = [r for r in rows if r[0] == "*"]
    assert len(chosen) == 1 and chosen[0][1] == "resident patch"
    assert "16-pixel blocks" in chosen[0][2]
    assert float(chosen[0][7]) == min(float(r[7]) for r in rows)
    # a layer of many tiles: rounds of 112-pixel tiles (measured 60 us against
    # 68 us for two streaming workgroups per CU)
    big = make_params(pa.HALF, batch=256, field=(14, 14), kernel=(3, 3),
                      ci=256, co=256, pad=1)
    text = pa.Plan(big).describe()
    assert "* resident patch 112 x 128, 16-pixel blocks" in text
    assert "896 on 256 CUs (256 busy, 4 round(s) of tiles)" in text
    assert "streaming 128 x 128, 2 stages" in text

    def forced(**kw):
        return pa.Plan(p, {"planConstraints":
                           json.dumps({"gfx950": kw})}).describe()
    assert "resident" not in forced(patch=0)
    assert "LDS stages                 4" in forced(patch=0)
    assert "* resident patch 64 x 128" in forced(patch=1, blockM=64)
    assert "392 on 256 CUs (256 busy, 2 round(s)" in forced(patch=1,
                                                             blockM=64)
    assert "* resident patch 128 x 128" in forced(patch=1)
    assert "196 on 256 CUs (196 busy, 1 round(s)" in forced(patch=1)
    assert "* resident patch 112 x 128, 16-pixel blocks" in forced(patch=2)
    assert "* resident patch 98 x 128, 16-pixel blocks" in \
        forced(patch=2, blockM=98)
    assert "* resident patch 112 x 128, 16-pixel blocks" in \
        forced(patch=2, blockM=112)
    with pytest.raises(MxconvError):
        forced(patch=2, blockM=113)
    assert "LDS stages                 2" in forced(stages=2)


def test_pointwise_planner_choice_for_padded_rows():
    """Rows padded to 256 channels go to the big tile on small layers."""
    def kernel_of(**kw):
        return pa.Plan(make_params(pa.HALF, kernel=(1, 1), **kw)).describe()
    assert "pointwise streaming variant" in kernel_of(
        batch=32, field=(56, 56), ci=144, co=24)
    assert "pointwise streaming variant" not in kernel_of(
        batch=32, field=(28, 28), ci=144, co=32)
    assert "pointwise streaming variant" in kernel_of(
        batch=32, field=(112, 112), ci=16, co=96)
    assert "pointwise streaming variant" in kernel_of(
        batch=32, field=(14, 14), ci=384, co=64)
    # not a multiple of eight: the big tile, channels padded in a copy
    assert "pointwise streaming variant" not in kernel_of(
        batch=2, field=(14, 14), ci=20, co=64)
    # fp8 inputs: rows of fewer than 512 bytes
    def quarter(**kw):
        return pa.Plan(make_params(pa.QUARTER, pa.HALF, kernel=(1, 1),
                                   **kw)).describe()
    assert "pointwise streaming variant" in quarter(
        batch=32, field=(56, 56), ci=256, co=64)
    assert "pointwise streaming variant" in quarter(
        batch=32, field=(112, 112), ci=32, co=64)
    assert "pointwise streaming variant" not in quarter(
        batch=32, field=(28, 28), ci=512, co=128)
    assert "pointwise streaming variant" not in quarter(
        batch=32, field=(28, 28), ci=24, co=128)


def test_planner_runs_small_conv_groups_as_one():
    """Groups of fewer input channels than half a 128-byte slice: the
    smallest number of groups that makes a whole slice runs as one."""
    import json

    def per_group(options=None, dtype=pa.HALF, out=None, **kw):
        text = pa.Plan(make_params(dtype, out, kernel=(3, 3), pad=1,
                                   batch=4, field=(14, 14), **kw),
                       options).describe()
        for line in text.splitlines():
            if "conv groups per group" in line:
                return int(line.split()[4])
        return 1
    assert per_group(ci=4, co=4, groups=32) == 16
    assert per_group(ci=8, co=8, groups=32) == 8
    assert per_group(ci=16, co=24, groups=12) == 4
    assert per_group(ci=24, co=24, groups=6) == 3
    assert per_group(dtype=pa.QUARTER, out=pa.HALF, ci=16, co=16,
                     groups=16) == 8
    # left alone: half a slice or more per group, depthwise, fused groups of
    # more than 256 output channels, too few groups for a whole slice
    assert per_group(ci=32, co=32, groups=8) == 1
    assert per_group(ci=1, co=1, groups=64) == 1
    # ... but a depthwise layer with a channel multiplier is not
    assert per_group(ci=1, co=2, groups=64) == 64
    assert per_group(ci=1, co=6, groups=64) == 1
    assert per_group(ci=4, co=64, groups=32) == 1
    # too few groups for a whole slice: all of them as one
    assert per_group(ci=4, co=4, groups=8) == 8
    assert per_group(ci=2, co=2, groups=4) == 1
    assert per_group({"pass": "TRAINING_BWD"}, ci=4, co=4, groups=32) == 16
    # the weight update pass of such a layer is planned for the layer with
    # the same groups taken as one
    layer = make_params(pa.HALF, batch=4, field=(14, 14), kernel=(3, 3), ci=4,
                        co=4, groups=32, pad=1)
    wu = pa.WeightUpdatePlan(layer).describe()
    assert "conv groups per group      16 (the weight update pass" in wu
    assert "numConvGroups              2" in wu
    assert "conv groups per group" not in pa.WeightUpdatePlan(
        make_params(pa.HALF, batch=4, field=(14, 14), kernel=(3, 3), ci=32,
                    co=32, groups=8, pad=1)).describe()
    # the reference's constraint, where it can be taken
    def forced(n):
        return {"planConstraints": json.dumps({"convGroupsPerGroup": n})}
    assert per_group(forced(4), ci=4, co=4, groups=32) == 4
    assert per_group(forced(1), ci=4, co=4, groups=32) == 1
    assert per_group(forced(5), ci=4, co=4, groups=32) == 1
    assert per_group(forced(2), ci=32, co=32, groups=8) == 2
    # room for the block-diagonal weights behind the packed ones
    p = make_params(pa.HALF, batch=4, field=(14, 14), kernel=(3, 3), ci=4,
                    co=4, groups=32, pad=1)
    plan, alone = pa.Plan(p), pa.Plan(p, forced(1))
    external = 32 * 4 * 4 * 9 * 2
    assert plan.buffer_bytes(pa.capi.BUF_WEIGHTS_EXTERNAL) == external
    packed = 2 * 64 * 576 * 2
    assert plan.buffer_bytes(pa.capi.BUF_WEIGHTS_PACKED) == \
        packed + 16 * external
    assert not plan.packs_like(alone)


def test_depthwise_7x7_tiles_fill_the_workgroup():
    """7 x 7 taps at unit stride: a thread forms a strip of neighbouring
    pixels; the planner's tile keeps most of the 256 threads busy."""
    def tile(**kw):
        text = pa.Plan(make_params(pa.HALF, batch=32, kernel=(7, 7), pad=3,
                                   **kw)).describe()
        line = [l for l in text.splitlines() if "output tile H x W" in l][0]
        return " ".join(line.split()[5:])
    # 12 channel vectors x 7 rows x 3 strips of 4 = 252 threads
    assert tile(field=(56, 56), groups=96) == \
        "7 x 12, a strip of 4 neighbouring pixels per thread"
    # 16 x 7 x 2 strips of 7 = 224
    assert tile(field=(14, 14), groups=384) == \
        "7 x 14, a strip of 7 neighbouring pixels per thread"
    # a 7 x 7 field: two strips of four (224 threads) rather than one of
    # seven (112)
    assert tile(field=(7, 7), groups=768) == \
        "7 x 7, a strip of 4 neighbouring pixels per thread"
    # strided or dilated 7 x 7, and other kernels: a pixel at a time
    assert "strip" not in tile(field=(28, 28), groups=64, stride=2)
    assert "strip" not in pa.Plan(make_params(
        pa.HALF, batch=4, field=(28, 28), kernel=(9, 9), groups=64,
        pad=4)).describe()
    # a forced tile keeps the strips; one that does not fit is refused
    forced = pa.Plan(make_params(pa.HALF, batch=4, field=(28, 28),
                                 kernel=(7, 7), groups=64, pad=3),
                     {"planConstraints":
                      '{"gfx950": {"tileH": 5, "tileW": 14}}'}).describe()
    assert "5 x 14, a strip of 4 neighbouring pixels" in forced
    with pytest.raises(MxconvError):
        pa.Plan(make_params(pa.HALF, batch=4, field=(64, 64), kernel=(7, 7),
                            groups=128, pad=3),
                {"planConstraints": '{"gfx950": {"tileH": 32, "tileW": 16}}'})

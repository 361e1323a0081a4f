"""Known-answer test at the level of PopLibs' AMP 1x1 vertex.

The reference's codelet test (tests/poplin/codelets/ConvPartial1x1Out.cpp)
fills its tensors with closed-form data (populateData, :175-203:
in[i][j] = i * 0.27182818 - j * 0.31415926,
weights[i][j] = i * 0.142857 - j * 0.0618034) and checks the device against a
host restatement of the vertex (vertexCompute, :101-163).  Here that
restatement is written again for dense work lists (every field element, no
flipped output), fed the same closed-form data, and its result must be what
the oracle - and the GPU - give for the 1x1 convolution the vertex data
describe:
  in      [cg * IG + ig][f * ICg + ic]
  weights [cg * OG * IG + ig * OG + (OG - 1 - og)][oc * ICg + ic]
  out     [cg * OG + og][f * OCg + oc]   (first in-group sets, later ones add)
"""
import numpy as np
import pytest

import poplibs_amd as pa
from helpers import rel_l2

CG, OG, IG, OCG, ICG, FIELD = 2, 2, 2, 8, 16, 24


def _populate():
    i, j = np.meshgrid(np.arange(CG * IG), np.arange(FIELD * ICG),
                       indexing="ij")
    vin = (i * 0.27182818 - j * 0.31415926).astype(np.float32)
    i, j = np.meshgrid(np.arange(CG * OG * IG), np.arange(OCG * ICG),
                       indexing="ij")
    vw = (i * 0.142857 - j * 0.0618034).astype(np.float32)
    return vin, vw


def _vertex_compute(vin, vw):
    """vertexCompute with work lists that cover every field element in order
    (outOffset = inOffset = 0, inStride = 1, flipOut = false): float sums, the
    first input channel group sets the output, the others accumulate."""
    out = np.zeros((CG * OG, FIELD * OCG), dtype=np.float32)
    for cg in range(CG):
        for og in range(OG):
            out_row = cg * OG + og
            for ig in range(IG):
                w_row = cg * OG * IG + ig * OG + (OG - 1 - og)
                in_row = cg * IG + ig
                for f in range(FIELD):
                    for oc in range(OCG):
                        s = np.float32(0)
                        for ic in range(ICG):
                            s = np.float32(s + vin[in_row, f * ICG + ic]
                                           * vw[w_row, oc * ICG + ic])
                        if ig == 0:
                            out[out_row, f * OCG + oc] = s
                        else:
                            out[out_row, f * OCG + oc] += s
    return out


def _as_convolution(vin, vw):
    """The vertex tensors in the external convolution layouts."""
    ci, co = IG * ICG, OG * OCG
    acts = np.zeros((1, CG * ci, FIELD))
    weights = np.zeros((CG, co, ci, 1))
    for cg in range(CG):
        for ig in range(IG):
            block = vin[cg * IG + ig].reshape(FIELD, ICG)
            acts[0, cg * ci + ig * ICG:cg * ci + (ig + 1) * ICG, :] = block.T
            for og in range(OG):
                w_row = cg * OG * IG + ig * OG + (OG - 1 - og)
                weights[cg, og * OCG:(og + 1) * OCG,
                        ig * ICG:(ig + 1) * ICG, 0] = \
                    vw[w_row].reshape(OCG, ICG)
    p = pa.ConvParams(pa.FLOAT, pa.FLOAT, 1, [FIELD], [1], ci, co, CG)
    return p, acts, weights


def _vertex_layout(conv_out):
    """[1][cg * Co + og * OCg + oc][f] -> [cg * OG + og][f * OCg + oc]."""
    co = OG * OCG
    out = np.zeros((CG * OG, FIELD * OCG))
    for cg in range(CG):
        for og in range(OG):
            block = conv_out[0, cg * co + og * OCG:cg * co + (og + 1) * OCG, :]
            out[cg * OG + og] = block.T.reshape(-1)
    return out


def test_oracle_reproduces_the_vertex_restatement(oracle):
    vin, vw = _populate()
    want = _vertex_compute(vin, vw)
    p, acts, weights = _as_convolution(vin, vw)
    got = _vertex_layout(oracle.convolution(p, acts, weights))
    # float32 running sums against double ones
    assert rel_l2(got, want.astype(np.float64)) <= 1e-6
    # a dropped in-group, a transposed operand or the un-reversed weight row
    # order would be off by tens of percent
    assert np.abs(want).max() > 100


@pytest.mark.gpu
@pytest.mark.parametrize("kernel", ["igemm", "generic"])
def test_gpu_reproduces_the_vertex_restatement(oracle, kernel):
    from gpu_helpers import run_conv
    vin, vw = _populate()
    want = _vertex_compute(vin, vw)
    p, acts, weights = _as_convolution(vin, vw)
    opts = {"planConstraints": '{"gfx950": {"kernel": "%s"}}' % kernel}
    got = run_conv(p, acts.astype(np.float32), weights.astype(np.float32),
                   None, opts)
    assert rel_l2(_vertex_layout(got), want.astype(np.float64)) <= 1e-5

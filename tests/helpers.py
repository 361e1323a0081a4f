"""Shared test utilities: seeded parameter/data generation and an independent
index-definition convolution used to pin the oracle."""
import itertools
import random

import numpy as np

import poplibs_amd as pa

NONE = 0xFFFFFFFF


def make_params(dtype=pa.FLOAT, out_dtype=None, batch=1, field=(4, 4),
                kernel=(3, 3), ci=1, co=1, groups=1, **kw):
    """ConvParams with keyword shortcuts: stride, pad (lower=upper), padLower,
    padUpper, kdil, idil, itl/itu (input truncation), ktl/ktu, kpl/kpu,
    flipIn, flipK, otl/otu, opl/opu."""
    n = len(field)
    p = pa.ConvParams(dtype, out_dtype, batch, list(field), list(kernel), ci,
                      co, groups)

    def vec(v):
        return [v] * n if isinstance(v, (int, bool)) else list(v)

    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    if "pad" in kw:
        it.paddingLower = vec(kw["pad"])
        it.paddingUpper = vec(kw["pad"])
    for key, obj, attr in (
            ("padLower", it, "paddingLower"), ("padUpper", it, "paddingUpper"),
            ("idil", it, "dilation"), ("itl", it, "truncationLower"),
            ("itu", it, "truncationUpper"), ("flipIn", it, "flip"),
            ("kdil", kt, "dilation"), ("ktl", kt, "truncationLower"),
            ("ktu", kt, "truncationUpper"), ("kpl", kt, "paddingLower"),
            ("kpu", kt, "paddingUpper"), ("flipK", kt, "flip"),
            ("stride", ot, "stride"), ("otl", ot, "truncationLower"),
            ("otu", ot, "truncationUpper"), ("opl", ot, "paddingLower"),
            ("opu", ot, "paddingUpper")):
        if key in kw:
            setattr(obj, attr, vec(kw[key]))
    return p


# ---------------------------------------------------------------------------
# Second, independent statement of the convolution semantics: the closed-form
# per-dimension index map of poplin::getInputIndex
# (lib/poplin/ConvUtil.cpp:95-268), written here in Python from that
# definition.  The oracle instead materialises the transformed arrays
# (lib/poplibs_test/Convolution.cpp:125-195); agreement of the two pins both.

def _dilated(size, dilation):
    return 0 if size == 0 else 1 + (size - 1) * dilation


def _forward(index, size, tl, tu, dil, pl, pu, flip):
    if index < tl or index >= size - tu:
        return None
    total = pl + _dilated(size - tl - tu, dil) + pu
    padded = (index - tl) * dil + pl
    return total - 1 - padded if flip else padded


def _backward(tindex, size, tl, tu, dil, pl, pu, flip):
    total = pl + _dilated(size - tl - tu, dil) + pu
    padded = total - 1 - tindex if flip else tindex
    if padded < pl or padded >= total - pu:
        return None
    d = padded - pl
    if d % dil:
        return None
    return d // dil + tl


def output_size_def(p, dim):
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    tin = (it.paddingLower[dim] + it.paddingUpper[dim] + _dilated(
        p.inputFieldShape[dim] - it.truncationLower[dim]
        - it.truncationUpper[dim], it.dilation[dim]))
    tk = (kt.paddingLower[dim] + kt.paddingUpper[dim] + _dilated(
        p.kernelShape[dim] - kt.truncationLower[dim]
        - kt.truncationUpper[dim], kt.dilation[dim]))
    conv = tin - tk + 1 - ot.truncationLower[dim] - ot.truncationUpper[dim]
    s = ot.stride[dim]
    return ot.paddingLower[dim] + (conv + s - 1) // s + ot.paddingUpper[dim]


def input_index_def(p, dim, o, k):
    """Input index multiplied with kernel index k for output o, or None."""
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    pk = _forward(k, p.kernelShape[dim], kt.truncationLower[dim],
                  kt.truncationUpper[dim], kt.dilation[dim],
                  kt.paddingLower[dim], kt.paddingUpper[dim], kt.flip[dim])
    if pk is None:
        return None
    osize = output_size_def(p, dim)
    if o < ot.paddingLower[dim] or o >= osize - ot.paddingUpper[dim]:
        return None
    conv = (o - ot.paddingLower[dim]) * ot.stride[dim] + ot.truncationLower[dim]
    return _backward(pk + conv, p.inputFieldShape[dim],
                     it.truncationLower[dim], it.truncationUpper[dim],
                     it.dilation[dim], it.paddingLower[dim],
                     it.paddingUpper[dim], it.flip[dim])


def conv_by_index_definition(p, acts, weights, biases=None):
    """Direct summation using input_index_def; float64; small inputs only."""
    n = len(p.inputFieldShape)
    G, Ci, Co, B = (p.numConvGroups, p.inputChannelsPerConvGroup,
                    p.outputChannelsPerConvGroup, p.batchSize)
    out_field = [output_size_def(p, d) for d in range(n)]
    out = np.zeros((B, G * Co, *out_field))
    # per dimension table [o][k] -> input index or -1
    tables = []
    for d in range(n):
        t = np.full((out_field[d], p.kernelShape[d]), -1, dtype=np.int64)
        for o in range(out_field[d]):
            for k in range(p.kernelShape[d]):
                i = input_index_def(p, d, o, k)
                if i is not None:
                    t[o, k] = i
        tables.append(t)
    for o in itertools.product(*[range(s) for s in out_field]):
        for k in itertools.product(*[range(s) for s in p.kernelShape]):
            idx = [tables[d][o[d], k[d]] for d in range(n)]
            if any(i < 0 for i in idx):
                continue
            a = acts[(slice(None), slice(None), *idx)].reshape(B, G, Ci)
            w = weights[(slice(None), slice(None), slice(None), *k)]  # G,Co,Ci
            out[(slice(None), slice(None), *o)] += np.einsum(
                "bgi,goi->bgo", a, w).reshape(B, G * Co)
    if biases is not None:
        out += np.asarray(biases).reshape((1, -1) + (1,) * n)
    return out


# ---------------------------------------------------------------------------
# Seeded random parameters (tiny, for pinning and GPU parity).

def random_params(rng, dtype=pa.FLOAT, out_dtype=None, max_dims=3,
                  max_field=7, simple=False):
    """A valid random ConvParams exercising every transform.  `rng` is a
    random.Random."""
    for _ in range(1000):
        n = rng.randint(1, max_dims)
        field = [rng.randint(1, max_field) for _ in range(n)]
        kernel = [rng.randint(1, 4) for _ in range(n)]
        p = pa.ConvParams(dtype, out_dtype, rng.randint(1, 3), field, kernel,
                          rng.randint(1, 4), rng.randint(1, 4),
                          rng.randint(1, 3))
        it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform

        def maybe(hi, prob=0.35):
            return rng.randint(1, hi) if rng.random() < prob else 0

        for d in range(n):
            it.paddingLower[d] = maybe(3)
            it.paddingUpper[d] = maybe(3)
            ot.stride[d] = 1 + maybe(2)
            kt.dilation[d] = 1 + maybe(2)
            if not simple:
                it.truncationLower[d] = maybe(2, 0.2)
                it.truncationUpper[d] = maybe(2, 0.2)
                it.dilation[d] = 1 + maybe(2, 0.25)
                it.flip[d] = rng.random() < 0.2
                kt.truncationLower[d] = maybe(1, 0.15)
                kt.truncationUpper[d] = maybe(1, 0.15)
                kt.paddingLower[d] = maybe(2, 0.15)
                kt.paddingUpper[d] = maybe(2, 0.15)
                kt.flip[d] = rng.random() < 0.2
                ot.truncationLower[d] = maybe(2, 0.2)
                ot.truncationUpper[d] = maybe(2, 0.2)
                ot.paddingLower[d] = maybe(2, 0.2)
                ot.paddingUpper[d] = maybe(2, 0.2)
        try:
            p.validate()
        except pa.MxconvError:
            continue
        return p
    raise RuntimeError("could not draw valid parameters")


def random_data(p, seed, dist="uniform"):
    """Seeded activations [B][G*Ci][field], weights [G][Co][Ci][kernel] and
    biases in float64."""
    g = np.random.default_rng(seed)
    ashape = (p.batchSize, p.numConvGroups * p.inputChannelsPerConvGroup,
              *p.inputFieldShape)
    wshape = (p.numConvGroups, p.outputChannelsPerConvGroup,
              p.inputChannelsPerConvGroup, *p.kernelShape)
    nb = p.numConvGroups * p.outputChannelsPerConvGroup
    if dist == "pm1":  # the reference harness's exact +-1 mode
        return (g.choice([-1.0, 1.0], size=ashape),
                g.choice([-1.0, 1.0], size=wshape),
                g.choice([-1.0, 1.0], size=nb))
    if dist == "normal":
        return (g.standard_normal(ashape), g.standard_normal(wshape),
                g.standard_normal(nb))
    return (g.uniform(-1, 1, ashape), g.uniform(-1, 1, wshape),
            g.uniform(-1, 1, nb))


def rel_l2(actual, expected):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    denom = np.linalg.norm(expected.ravel())
    num = np.linalg.norm((actual - expected).ravel())
    return num / denom if denom > 0 else num


__all__ = [n for n in dir() if not n.startswith("_")]
_ = random

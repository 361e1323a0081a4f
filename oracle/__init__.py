"""ctypes binding of the CPU oracle (test infrastructure, not product code).

Only the tests, the smoke check and the benchmark's CPU-baseline leg import
this module.  The library is built by ``make -C oracle`` (also run by
``__graft_entry__.build``); nothing here falls back to another implementation
when it is missing.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libconv_oracle.so")
_lib = None


def build(force=False):
    """Compile conv_oracle.c into libconv_oracle.so."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "libconv_oracle.so"],
                          stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        u = ctypes.c_uint
        pu = ctypes.POINTER(ctypes.c_uint)
        pb = ctypes.POINTER(ctypes.c_ubyte)
        pd = ctypes.POINTER(ctypes.c_double)
        L.oracle_convolution.restype = ctypes.c_int
        L.oracle_convolution.argtypes = (
            [u, pu, pu, pu, pu, pu, pu, pb]      # input field + transform
            + [pu, pu, pu, pu, pu, pu, pb]       # kernel + transform
            + [pu, pu, pu, pu, pu]               # output transform
            + [u, u, u, u, pd, pd, pd, pd, ctypes.c_size_t, ctypes.c_int])
        L.oracle_convolution_backward.restype = ctypes.c_int
        L.oracle_convolution_backward.argtypes = (
            [u, pu, pu, pu, pu, pu, pu, pb]      # input field + transform
            + [pu, pu, pu, pu, pu, pu, pb]       # kernel + transform
            + [pu, pu, pu, pu, pu]               # output transform
            + [u, u, u, u, pd, pd, pd, ctypes.c_size_t, ctypes.c_int])
        L.oracle_weight_update.restype = ctypes.c_int
        L.oracle_weight_update.argtypes = (
            [u, pu, pu, pu, pu, pu, pu, pb]      # input field + transform
            + [pu, pu, pu, pu, pu, pu, pb]       # kernel + transform
            + [pu, pu, pu, pu, pu]               # output transform
            + [u, u, u, u, pd, pd, pd, ctypes.c_size_t, pd, ctypes.c_int])
        L.oracle_output_field_size.restype = u
        L.oracle_output_field_size.argtypes = [u] * 17
        L.oracle_fp8_decode.restype = ctypes.c_double
        L.oracle_fp8_decode.argtypes = [u, ctypes.c_int]
        L.oracle_fp8_encode.restype = u
        L.oracle_fp8_encode.argtypes = [ctypes.c_double, ctypes.c_int]
        L.oracle_quarter_metadata.restype = u
        L.oracle_quarter_metadata.argtypes = [ctypes.c_int, ctypes.c_int]
        L.oracle_quarter_to_double.restype = None
        L.oracle_quarter_to_double.argtypes = [pb, ctypes.c_size_t, u, pd]
        _lib = L
    return _lib


def _uarr(values):
    values = [int(v) for v in values]
    return (ctypes.c_uint * max(len(values), 1))(*values)


def _barr(values):
    values = [1 if v else 0 for v in values]
    return (ctypes.c_ubyte * max(len(values), 1))(*values)


def output_field_shape(p):
    """Output field shape by the oracle's own size arithmetic
    (lib/poplibs_test/Convolution.cpp:55-110)."""
    L = lib()
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    return [
        L.oracle_output_field_size(
            p.inputFieldShape[d], p.kernelShape[d], it.truncationLower[d],
            it.truncationUpper[d], it.dilation[d], it.paddingLower[d],
            it.paddingUpper[d], kt.truncationLower[d], kt.truncationUpper[d],
            kt.dilation[d], kt.paddingLower[d], kt.paddingUpper[d],
            ot.truncationLower[d], ot.truncationUpper[d], ot.stride[d],
            ot.paddingLower[d], ot.paddingUpper[d])
        for d in range(len(p.inputFieldShape))
    ]


def convolution(p, acts, weights, biases=None, threads=1):
    """Forward convolution in double precision.

    ``p`` is any object with the field names of poplin::ConvParams.
    ``acts`` has shape [B][G*Ci][field...], ``weights`` [G][Co][Ci][kernel...]
    (the external layouts of include/poplin/Convolution.hpp:323-328); the
    result has shape [B][G*Co][outField...], dtype float64.
    """
    L = lib()
    nd = len(p.inputFieldShape)
    G, Ci, Co, B = (p.numConvGroups, p.inputChannelsPerConvGroup,
                    p.outputChannelsPerConvGroup, p.batchSize)
    acts = np.ascontiguousarray(acts, dtype=np.float64)
    weights = np.ascontiguousarray(weights, dtype=np.float64)
    assert acts.shape == (B, G * Ci, *p.inputFieldShape), acts.shape
    assert weights.shape == (G, Co, Ci, *p.kernelShape), weights.shape
    if biases is None:
        biases = np.zeros(G * Co)
    biases = np.ascontiguousarray(biases, dtype=np.float64)
    assert biases.shape == (G * Co,)
    out_field = output_field_shape(p)
    out = np.empty((B, G * Co, *out_field), dtype=np.float64)
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    pd = ctypes.POINTER(ctypes.c_double)
    # Zero-sized arrays have no storage to point at; one spare double stands in.
    spare = np.zeros(1)

    def ptr(a):
        return (a if a.size else spare).ctypes.data_as(pd)

    rc = L.oracle_convolution(
        nd, _uarr(p.inputFieldShape), _uarr(it.truncationLower),
        _uarr(it.truncationUpper), _uarr(it.dilation), _uarr(it.paddingLower),
        _uarr(it.paddingUpper), _barr(it.flip),
        _uarr(p.kernelShape), _uarr(kt.truncationLower),
        _uarr(kt.truncationUpper), _uarr(kt.dilation), _uarr(kt.paddingLower),
        _uarr(kt.paddingUpper), _barr(kt.flip),
        _uarr(ot.truncationLower), _uarr(ot.truncationUpper), _uarr(ot.stride),
        _uarr(ot.paddingLower), _uarr(ot.paddingUpper),
        B, G, Ci, Co, ptr(acts), ptr(weights), ptr(biases), ptr(out),
        out.size, int(threads))
    if rc != 0:
        raise RuntimeError(f"oracle_convolution failed with code {rc}")
    return out


def convolution_backward(p, deltas, weights, threads=1):
    """Gradient of the forward convolution ``p`` with respect to its input.

    ``p`` describes the FORWARD pass.  ``deltas`` has the shape of the forward
    output [B][G*Co][outField...], ``weights`` are the forward weights
    [G][Co][Ci][kernel...]; the result has the shape of the forward input
    [B][G*Ci][field...], dtype float64.
    """
    L = lib()
    nd = len(p.inputFieldShape)
    G, Ci, Co, B = (p.numConvGroups, p.inputChannelsPerConvGroup,
                    p.outputChannelsPerConvGroup, p.batchSize)
    deltas = np.ascontiguousarray(deltas, dtype=np.float64)
    weights = np.ascontiguousarray(weights, dtype=np.float64)
    assert deltas.shape == (B, G * Co, *output_field_shape(p)), deltas.shape
    assert weights.shape == (G, Co, Ci, *p.kernelShape), weights.shape
    out = np.empty((B, G * Ci, *p.inputFieldShape), dtype=np.float64)
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    pd = ctypes.POINTER(ctypes.c_double)
    spare = np.zeros(1)

    def ptr(a):
        return (a if a.size else spare).ctypes.data_as(pd)

    rc = L.oracle_convolution_backward(
        nd, _uarr(p.inputFieldShape), _uarr(it.truncationLower),
        _uarr(it.truncationUpper), _uarr(it.dilation), _uarr(it.paddingLower),
        _uarr(it.paddingUpper), _barr(it.flip),
        _uarr(p.kernelShape), _uarr(kt.truncationLower),
        _uarr(kt.truncationUpper), _uarr(kt.dilation), _uarr(kt.paddingLower),
        _uarr(kt.paddingUpper), _barr(kt.flip),
        _uarr(ot.truncationLower), _uarr(ot.truncationUpper), _uarr(ot.stride),
        _uarr(ot.paddingLower), _uarr(ot.paddingUpper),
        B, G, Ci, Co, ptr(deltas), ptr(weights), ptr(out), out.size,
        int(threads))
    if rc != 0:
        raise RuntimeError(f"oracle_convolution_backward failed with code {rc}")
    return out


def weight_deltas(p, activations, deltas, threads=1, with_bias=False):
    """Gradient of the forward convolution ``p`` with respect to its weights
    (and, with ``with_bias``, its biases): the deltas that
    poplibs_test::conv::weightUpdate scales by -learningRate and adds.

    ``activations`` [B][G*Ci][field...] are the forward input, ``deltas``
    [B][G*Co][outField...] the gradient of the forward output; the result is
    [G][Co][Ci][kernel...] (and [G*Co]), dtype float64.
    """
    L = lib()
    nd = len(p.inputFieldShape)
    G, Ci, Co, B = (p.numConvGroups, p.inputChannelsPerConvGroup,
                    p.outputChannelsPerConvGroup, p.batchSize)
    activations = np.ascontiguousarray(activations, dtype=np.float64)
    deltas = np.ascontiguousarray(deltas, dtype=np.float64)
    assert activations.shape == (B, G * Ci, *p.inputFieldShape), \
        activations.shape
    assert deltas.shape == (B, G * Co, *output_field_shape(p)), deltas.shape
    out = np.empty((G, Co, Ci, *p.kernelShape), dtype=np.float64)
    bias = np.empty(G * Co, dtype=np.float64)
    it, kt, ot = p.inputTransform, p.kernelTransform, p.outputTransform
    pd = ctypes.POINTER(ctypes.c_double)
    spare = np.zeros(1)

    def ptr(a):
        return (a if a.size else spare).ctypes.data_as(pd)

    rc = L.oracle_weight_update(
        nd, _uarr(p.inputFieldShape), _uarr(it.truncationLower),
        _uarr(it.truncationUpper), _uarr(it.dilation), _uarr(it.paddingLower),
        _uarr(it.paddingUpper), _barr(it.flip),
        _uarr(p.kernelShape), _uarr(kt.truncationLower),
        _uarr(kt.truncationUpper), _uarr(kt.dilation), _uarr(kt.paddingLower),
        _uarr(kt.paddingUpper), _barr(kt.flip),
        _uarr(ot.truncationLower), _uarr(ot.truncationUpper), _uarr(ot.stride),
        _uarr(ot.paddingLower), _uarr(ot.paddingUpper),
        B, G, Ci, Co, ptr(activations), ptr(deltas), ptr(out), out.size,
        ptr(bias), int(threads))
    if rc != 0:
        raise RuntimeError(f"oracle_weight_update failed with code {rc}")
    return (out, bias) if with_bias else out


def weight_update(p, learning_rate, activations, deltas, kernel, biases,
                  threads=1):
    """poplibs_test::conv::weightUpdate: returns the updated (kernel, biases),
    kernel - learning_rate * weight deltas and likewise for the biases
    (lib/poplibs_test/Convolution.cpp:870-897)."""
    dw, db = weight_deltas(p, activations, deltas, threads, with_bias=True)
    return (np.asarray(kernel, dtype=np.float64) + learning_rate * -dw,
            np.asarray(biases, dtype=np.float64) + learning_rate * -db)


E5M2, E4M3 = 0, 1


def fp8_decode_table(fmt):
    L = lib()
    return np.array([L.oracle_fp8_decode(c, fmt) for c in range(256)])


def fp8_encode(values, fmt):
    L = lib()
    flat = np.asarray(values, dtype=np.float64).ravel()
    out = np.fromiter((L.oracle_fp8_encode(float(v), fmt) for v in flat),
                      dtype=np.uint8, count=flat.size)
    return out.reshape(np.shape(values))


def quarter_metadata(fmt, scale):
    return lib().oracle_quarter_metadata(fmt, scale)


def quarter_to_double(codes, metadata):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape, dtype=np.float64)
    lib().oracle_quarter_to_double(
        codes.ctypes.data_as(ctypes.POINTER(ctypes.c_ubyte)), codes.size,
        metadata, out.ctypes.data_as(ctypes.POINTER(ctypes.c_double)))
    return out

"""Runs a convolution on the GPU through the C ABI.  torch is used only to
own device memory and move bytes; every computation is an mxconv_* call."""
import numpy as np
import torch

import poplibs_amd as pa
from poplibs_amd import capi

_TORCH_DTYPE = {pa.FLOAT: torch.float32, pa.HALF: torch.float16,
                pa.QUARTER: torch.uint8}
_NP_DTYPE = {pa.FLOAT: np.float32, pa.HALF: np.float16, pa.QUARTER: np.uint8}


def quantize(values, type_id, oracle=None, fmt=1, scale=0):
    """float64 -> (array in the device element type, the same values as
    float64 for the oracle)."""
    values = np.asarray(values, dtype=np.float64)
    if type_id == pa.QUARTER:
        codes = oracle.fp8_encode(values / 2.0 ** scale, fmt)
        back = oracle.quarter_to_double(codes,
                                        oracle.quarter_metadata(fmt, scale))
        return codes, back
    q = values.astype(_NP_DTYPE[type_id])
    return q, q.astype(np.float64)


def device(array, type_id):
    t = torch.from_numpy(np.ascontiguousarray(array))
    assert t.dtype == _TORCH_DTYPE[type_id], (t.dtype, type_id)
    return t.cuda()


def run_conv(p, acts_q, weights_q, bias_q=None, options=None, plan=None,
             in_meta=0x80, w_meta=0x80, return_plan=False):
    """acts_q / weights_q / bias_q: numpy arrays already in the device element
    types and the external layouts.  Returns the output in the external layout
    [B][G*Co][field...] as float64."""
    plan = plan or pa.Plan(p, options)
    dev = torch.device("cuda:0")
    out_shape = (p.batchSize, p.getNumOutputChans(), *p.getOutputFieldShape())
    a_ext = device(acts_q, p.inputType)
    w_ext = device(weights_q, p.inputType)

    def buf(which, dtype):
        nbytes = plan.buffer_bytes(which)
        return torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)

    a_int = buf(capi.BUF_INPUT, None)
    w_pack = buf(capi.BUF_WEIGHTS_PACKED, None)
    o_int = buf(capi.BUF_OUTPUT, None)
    ws_bytes = plan.buffer_bytes(capi.BUF_WORKSPACE)
    ws = buf(capi.BUF_WORKSPACE, None)
    o_ext = torch.empty(out_shape, dtype=_TORCH_DTYPE[p.outputType],
                        device=dev)
    assert a_ext.numel() * a_ext.element_size() == plan.buffer_bytes(
        capi.BUF_INPUT)
    assert w_ext.numel() * w_ext.element_size() == plan.buffer_bytes(
        capi.BUF_WEIGHTS_EXTERNAL)
    assert o_ext.numel() * o_ext.element_size() == plan.buffer_bytes(
        capi.BUF_OUTPUT)
    bias_dev = None
    if bias_q is not None:
        bias_dev = device(bias_q, p.outputType)
    stream = torch.cuda.current_stream().cuda_stream
    plan.acts_to_internal(a_ext.data_ptr(), a_int.data_ptr(), stream)
    plan.pack_weights(w_ext.data_ptr(), w_pack.data_ptr(), stream)
    bias_ptr = bias_dev.data_ptr() if bias_dev is not None else None
    if p.inputType == pa.QUARTER:
        plan.fwd_quarter(a_int.data_ptr(), in_meta, w_pack.data_ptr(), w_meta,
                         o_int.data_ptr(), bias_ptr, ws.data_ptr(), ws_bytes,
                         stream)
    else:
        plan.fwd(a_int.data_ptr(), w_pack.data_ptr(), o_int.data_ptr(),
                 bias_ptr, ws.data_ptr(), ws_bytes, stream)
    plan.acts_to_external(o_int.data_ptr(), o_ext.data_ptr(), stream)
    torch.cuda.synchronize()
    out = o_ext.cpu().numpy().astype(np.float64)
    return (out, plan) if return_plan else out

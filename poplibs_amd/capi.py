"""ctypes declarations for include/mxconv.h and thin Python conveniences.

`ConvParams`, `InputTransform` and `OutputTransform` carry the field names of
poplin::ConvParams (include/poplin/ConvParams.hpp:16-224) so that tests read
like the reference's; they only marshal into `mxconv_params` - validation,
canonicalisation, size and range algebra all run in the C++ library.
"""
import ctypes
import os
import subprocess
from ctypes import (POINTER, Structure, byref, c_char_p, c_int, c_int32,
                    c_size_t, c_uint8, c_uint32, c_uint64, c_void_p)

MAX_FIELD_DIMS = 4
NO_INDEX = 0xFFFFFFFF
QUARTER, HALF, FLOAT = 0, 1, 2
TYPE_NAMES = {QUARTER: "quarter", HALF: "half", FLOAT: "float"}
TYPE_BYTES = {QUARTER: 1, HALF: 2, FLOAT: 4}


class Status:
    OK = 0
    INVALID_PARAMS = 1
    INVALID_OPTION = 2
    UNSUPPORTED = 3
    OUT_OF_MEMORY = 4
    WORKSPACE_TOO_SMALL = 5
    BUFFER_TOO_SMALL = 6
    HIP_ERROR = 7
    NULL_ARGUMENT = 8


class MxconvError(RuntimeError):
    """A failing C ABI call; `.status` is the mxconv_status value.

    INVALID_PARAMS corresponds to poputil::poplibs_error and INVALID_OPTION to
    poplar::invalid_option in the reference.
    """

    def __init__(self, status, message):
        super().__init__(f"mxconv status {status}: {message}")
        self.status = status
        self.message = message


_U32x = c_uint32 * MAX_FIELD_DIMS
_U64x = c_uint64 * MAX_FIELD_DIMS
_U8x = c_uint8 * MAX_FIELD_DIMS


class _CInputTransform(Structure):
    _fields_ = [("truncation_lower", _U32x), ("truncation_upper", _U32x),
                ("dilation", _U32x), ("padding_lower", _U32x),
                ("padding_upper", _U32x), ("flip", _U8x)]


class _COutputTransform(Structure):
    _fields_ = [("truncation_lower", _U32x), ("truncation_upper", _U32x),
                ("stride", _U32x), ("padding_lower", _U32x),
                ("padding_upper", _U32x)]


class CParams(Structure):
    _fields_ = [("input_type", c_int32), ("output_type", c_int32),
                ("num_field_dims", c_uint32), ("reserved", c_uint32),
                ("batch_size", c_uint64), ("input_field_shape", _U64x),
                ("kernel_shape", _U64x),
                ("input_channels_per_conv_group", c_uint64),
                ("output_channels_per_conv_group", c_uint64),
                ("num_conv_groups", c_uint64),
                ("input_transform", _CInputTransform),
                ("kernel_transform", _CInputTransform),
                ("output_transform", _COutputTransform)]


class _CPhaseCost(Structure):
    _fields_ = [("cycles", c_uint64), ("memory_bytes", c_uint64)]


class DetailedCosts(Structure):
    """mxconv_detailed_costs."""
    _fields_ = [("parallel_split", c_uint64), ("serial_split", c_uint64),
                ("rearrangement", _CPhaseCost), ("compute", _CPhaseCost),
                ("reduction", _CPhaseCost), ("total", _CPhaseCost)]


_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmxconv.so")
_lib = None


def library_path():
    return _LIB_PATH


def build_library(force=False):
    """Compile libmxconv.so for gfx950 (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", _HERE, "-j8", "all"]
    if force:
        cmd.insert(1, "-B")
    subprocess.check_call(cmd)


def lib():
    """The loaded C ABI library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    # A process must hold ONE HIP runtime.  PyTorch ships its own copy of
    # libamdhip64 (same soname as the system one); callers here use torch
    # tensors as device memory, so torch has to load first - the dynamic
    # loader then binds libmxconv.so's libamdhip64.so.7 to that copy instead of
    # mapping a second runtime that cannot see the first one's allocations.
    import torch  # noqa: F401
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with "
            "`python -c 'import __graft_entry__ as g; g.build()'` or "
            "`make -C poplibs_amd`. There is no fallback implementation.")
    L = ctypes.CDLL(_LIB_PATH)
    P = POINTER(CParams)
    sigs = {
        "mxconv_last_error": (c_char_p, []),
        "mxconv_status_string": (c_char_p, [c_int]),
        "mxconv_params_init": (c_int, [P, c_int32, c_int32, c_uint64, c_uint32,
                                       POINTER(c_uint64), POINTER(c_uint64),
                                       c_uint64, c_uint64, c_uint64]),
        "mxconv_params_validate": (c_int, [P]),
        "mxconv_params_canonicalize": (c_int, [P, P]),
        "mxconv_get_gradient_params": (c_int, [P, P]),
        "mxconv_get_weight_update_params": (c_int, [P, P]),
        "mxconv_weight_update_plan_create": (c_int, [P, POINTER(c_char_p),
                                                     POINTER(c_char_p),
                                                     c_size_t,
                                                     POINTER(c_void_p)]),
        "mxconv_weight_update_workspace_bytes": (c_int, [c_void_p,
                                                         POINTER(c_size_t)]),
        "mxconv_calculate_weight_deltas": (c_int, [c_void_p, c_void_p, c_void_p,
                                                   c_void_p, c_void_p,
                                                   c_size_t, c_void_p]),
        "mxconv_convolution_weight_update": (c_int, [c_void_p, c_void_p,
                                                     c_void_p, c_void_p,
                                                     ctypes.c_float, c_void_p,
                                                     c_size_t, c_void_p]),
        "mxconv_bias_update_workspace_bytes": (c_int, [c_uint64, c_uint64,
                                                       POINTER(c_size_t)]),
        "mxconv_convolution_bias_update": (c_int, [c_int32, c_void_p, c_uint64,
                                                   c_uint64, c_int32, c_void_p,
                                                   ctypes.c_float, c_void_p,
                                                   c_size_t, c_void_p]),
        "mxconv_weights_transpose_chans_flip_xy":
            (c_int, [P, c_void_p, c_void_p, c_void_p]),
        "mxconv_params_is_zero_convolution": (c_int, [P, POINTER(c_int)]),
        "mxconv_params_size": (c_int, [P, c_int32, c_uint32,
                                       POINTER(c_uint64)]),
        "mxconv_params_compare": (c_int, [P, P, POINTER(c_int)]),
        "mxconv_params_hash": (c_int, [P, POINTER(c_uint64)]),
        "mxconv_params_from_json": (c_int, [c_char_p, P]),
        "mxconv_params_to_string": (c_int, [P, c_char_p, c_size_t,
                                            POINTER(c_size_t)]),
        "mxconv_get_input_index": (c_int, [P, c_uint32, c_uint32, c_uint32,
                                           POINTER(c_uint32)]),
        "mxconv_get_kernel_index": (c_int, [P, c_uint32, c_uint32, c_uint32,
                                            POINTER(c_uint32)]),
        "mxconv_get_range": (c_int, [P, c_int32, c_uint32, POINTER(c_uint32),
                                     POINTER(c_uint32), POINTER(c_uint32)]),
        "mxconv_get_number_of_macs": (c_int, [P, POINTER(c_uint64)]),
        "mxconv_get_fwd_flops": (c_int, [P, POINTER(c_uint64)]),
        "mxconv_validate_options": (c_int, [POINTER(c_char_p),
                                            POINTER(c_char_p), c_size_t]),
        "mxconv_plan_create": (c_int, [P, POINTER(c_char_p), POINTER(c_char_p),
                                       c_size_t, POINTER(c_void_p)]),
        "mxconv_plan_destroy": (None, [c_void_p]),
        "mxconv_plan_describe": (c_int, [c_void_p, c_char_p, c_size_t,
                                         POINTER(c_size_t)]),
        "mxconv_plan_constraints": (c_int, [c_void_p, c_char_p, c_size_t,
                                         POINTER(c_size_t)]),
        "mxconv_plan_buffer_bytes": (c_int, [c_void_p, c_int32,
                                             POINTER(c_size_t)]),
        "mxconv_plan_estimated_costs": (c_int, [c_void_p, POINTER(c_uint64),
                                                POINTER(c_uint64)]),
        "mxconv_plan_detailed_costs": (c_int, [c_void_p,
                                               POINTER(DetailedCosts)]),
        "mxconv_plans_pack_alike": (c_int, [c_void_p, c_void_p,
                                            POINTER(c_int32)]),
        "mxconv_pack_weights": (c_int, [c_void_p, c_void_p, c_void_p,
                                        c_void_p]),
        "mxconv_acts_to_internal": (c_int, [c_void_p, c_void_p, c_void_p,
                                            c_void_p]),
        "mxconv_acts_to_external": (c_int, [c_void_p, c_void_p, c_void_p,
                                            c_void_p]),
        "mxconv_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_size_t, c_void_p]),
        "mxconv_fwd_static_scratch": (c_int, [c_void_p, c_void_p, c_void_p,
                                              c_void_p, c_void_p, c_void_p]),
        "mxconv_fwd_quarter": (c_int, [c_void_p, c_void_p, c_uint8, c_void_p,
                                       c_uint8, c_void_p, c_void_p, c_void_p,
                                       c_size_t, c_void_p]),
        "mxconv_multi_fwd": (c_int, [c_size_t, POINTER(c_void_p),
                                     POINTER(c_void_p), POINTER(c_uint8),
                                     POINTER(c_void_p), POINTER(c_uint8),
                                     POINTER(c_void_p), POINTER(c_void_p),
                                     POINTER(c_void_p), POINTER(c_size_t),
                                     c_int, c_void_p]),
        "mxconv_multiconv_validate_options": (c_int, [POINTER(c_char_p),
                                                      POINTER(c_char_p),
                                                      c_size_t,
                                                      POINTER(c_int)]),
        "mxconv_matmul_params": (c_int, [c_int32, c_int32, c_uint64, c_uint64,
                                         c_uint64, c_uint64, P]),
        "mxconv_matmul_validate_options": (c_int, [POINTER(c_char_p),
                                                   POINTER(c_char_p),
                                                   c_size_t]),
        "mxconv_matmul_plan_create": (c_int, [c_int32, c_int32, c_uint64,
                                              c_uint64, c_uint64, c_uint64,
                                              POINTER(c_char_p),
                                              POINTER(c_char_p), c_size_t,
                                              POINTER(c_void_p)]),
        "mxconv_matmul_pack_rhs": (c_int, [c_void_p, c_void_p, c_void_p,
                                           c_void_p]),
        "mxconv_matmul_lhs_to_internal": (c_int, [c_void_p, c_void_p, c_void_p,
                                                  c_void_p]),
        "mxconv_matmul_out_to_external": (c_int, [c_void_p, c_void_p, c_void_p,
                                                  c_void_p]),
        "mxconv_transpose_grouped_matrix": (c_int, [c_int32, c_uint64, c_uint64,
                                                    c_uint64, c_void_p,
                                                    c_void_p, c_void_p]),
        "mxconv_scaled_add_to": (c_int, [c_int32, c_void_p, ctypes.c_float,
                                         c_void_p, ctypes.c_float, c_uint64,
                                         c_void_p]),
        "mxconv_add_bias": (c_int, [c_int32, c_void_p, c_void_p, c_uint64,
                                    c_uint64, c_void_p]),
    }
    for name, (restype, argtypes) in sigs.items():
        fn = getattr(L, name)
        fn.restype = restype
        fn.argtypes = argtypes
    L._declared = sorted(sigs)
    _lib = L
    return L


def _check(status):
    if status != Status.OK:
        raise MxconvError(status, lib().mxconv_last_error().decode())


class InputTransform:
    def __init__(self, n=0, truncationLower=None, truncationUpper=None,
                 dilation=None, paddingLower=None, paddingUpper=None,
                 flip=None):
        self.truncationLower = list(truncationLower or [0] * n)
        self.truncationUpper = list(truncationUpper or [0] * n)
        self.dilation = list(dilation or [1] * n)
        self.paddingLower = list(paddingLower or [0] * n)
        self.paddingUpper = list(paddingUpper or [0] * n)
        self.flip = list(flip or [False] * n)

    def _fields(self):
        return (self.truncationLower, self.truncationUpper, self.dilation,
                self.paddingLower, self.paddingUpper, self.flip)

    def __eq__(self, o):
        return self._fields() == o._fields()

    def __repr__(self):
        return ("InputTransform(truncationLower=%r, truncationUpper=%r, "
                "dilation=%r, paddingLower=%r, paddingUpper=%r, flip=%r)"
                % self._fields())


class OutputTransform:
    def __init__(self, n=0, truncationLower=None, truncationUpper=None,
                 stride=None, paddingLower=None, paddingUpper=None):
        self.truncationLower = list(truncationLower or [0] * n)
        self.truncationUpper = list(truncationUpper or [0] * n)
        self.stride = list(stride or [1] * n)
        self.paddingLower = list(paddingLower or [0] * n)
        self.paddingUpper = list(paddingUpper or [0] * n)

    def _fields(self):
        return (self.truncationLower, self.truncationUpper, self.stride,
                self.paddingLower, self.paddingUpper)

    def __eq__(self, o):
        return self._fields() == o._fields()

    def __repr__(self):
        return ("OutputTransform(truncationLower=%r, truncationUpper=%r, "
                "stride=%r, paddingLower=%r, paddingUpper=%r)" % self._fields())


class ConvParams:
    """Mirror of poplin::ConvParams; see the module docstring."""

    def __init__(self, inputType, outputType=None, batchSize=1,
                 inputFieldShape=(), kernelShape=(),
                 inputChannelsPerConvGroup=1, outputChannelsPerConvGroup=1,
                 numConvGroups=1, inputTransform=None, kernelTransform=None,
                 outputTransform=None):
        n = len(inputFieldShape)
        self.inputType = inputType
        self.outputType = inputType if outputType is None else outputType
        self.batchSize = batchSize
        self.inputFieldShape = list(inputFieldShape)
        self.kernelShape = list(kernelShape)
        self.inputChannelsPerConvGroup = inputChannelsPerConvGroup
        self.outputChannelsPerConvGroup = outputChannelsPerConvGroup
        self.numConvGroups = numConvGroups
        self.inputTransform = inputTransform or InputTransform(n)
        self.kernelTransform = kernelTransform or InputTransform(n)
        self.outputTransform = outputTransform or OutputTransform(n)

    # -- marshalling ------------------------------------------------------
    def to_c(self):
        n = len(self.inputFieldShape)
        if n > MAX_FIELD_DIMS:
            raise MxconvError(Status.INVALID_PARAMS,
                              "too many field dimensions")
        c = CParams()
        c.input_type, c.output_type = self.inputType, self.outputType
        c.num_field_dims = n
        c.batch_size = self.batchSize
        c.input_channels_per_conv_group = self.inputChannelsPerConvGroup
        c.output_channels_per_conv_group = self.outputChannelsPerConvGroup
        c.num_conv_groups = self.numConvGroups
        if len(self.kernelShape) != n:
            raise MxconvError(
                Status.INVALID_PARAMS,
                "Number of kernel field dimensions does not match the number "
                "of input field dimensions")
        for d in range(n):
            c.input_field_shape[d] = self.inputFieldShape[d]
            c.kernel_shape[d] = self.kernelShape[d]

        def put(dst, src, what):
            if len(src) != n:
                raise MxconvError(
                    Status.INVALID_PARAMS,
                    f"Number of {what} dimensions ({len(src)}) does not match "
                    f"the number of field dimensions ({n})")
            for d in range(n):
                dst[d] = int(src[d])

        for ct, t, name in ((c.input_transform, self.inputTransform, "input"),
                            (c.kernel_transform, self.kernelTransform,
                             "kernel")):
            put(ct.truncation_lower, t.truncationLower, name + " truncation")
            put(ct.truncation_upper, t.truncationUpper, name + " truncation")
            put(ct.dilation, t.dilation, name + " dilation")
            put(ct.padding_lower, t.paddingLower, name + " padding")
            put(ct.padding_upper, t.paddingUpper, name + " padding")
            put(ct.flip, t.flip, name + " flip")
        ot, o = c.output_transform, self.outputTransform
        put(ot.truncation_lower, o.truncationLower, "output truncation")
        put(ot.truncation_upper, o.truncationUpper, "output truncation")
        put(ot.stride, o.stride, "stride")
        put(ot.padding_lower, o.paddingLower, "output padding")
        put(ot.padding_upper, o.paddingUpper, "output padding")
        return c

    @staticmethod
    def from_c(c):
        n = c.num_field_dims

        def it(t):
            return InputTransform(
                n, list(t.truncation_lower[:n]), list(t.truncation_upper[:n]),
                list(t.dilation[:n]), list(t.padding_lower[:n]),
                list(t.padding_upper[:n]), [bool(f) for f in t.flip[:n]])

        o = c.output_transform
        return ConvParams(
            c.input_type, c.output_type, c.batch_size,
            list(c.input_field_shape[:n]), list(c.kernel_shape[:n]),
            c.input_channels_per_conv_group, c.output_channels_per_conv_group,
            c.num_conv_groups, it(c.input_transform), it(c.kernel_transform),
            OutputTransform(n, list(o.truncation_lower[:n]),
                            list(o.truncation_upper[:n]), list(o.stride[:n]),
                            list(o.padding_lower[:n]),
                            list(o.padding_upper[:n])))

    @staticmethod
    def from_json(text):
        c = CParams()
        _check(lib().mxconv_params_from_json(text.encode(), byref(c)))
        return ConvParams.from_c(c)

    def _fields(self):
        return (self.inputType, self.outputType, self.batchSize,
                self.inputFieldShape, self.kernelShape,
                self.inputChannelsPerConvGroup,
                self.outputChannelsPerConvGroup, self.numConvGroups)

    def __eq__(self, o):
        return (self._fields() == o._fields()
                and self.inputTransform == o.inputTransform
                and self.kernelTransform == o.kernelTransform
                and self.outputTransform == o.outputTransform)

    def __repr__(self):
        return ("ConvParams(%s->%s, batch=%d, field=%r, kernel=%r, Ci=%d, "
                "Co=%d, G=%d, in=%r, k=%r, out=%r)" % (
                    TYPE_NAMES[self.inputType], TYPE_NAMES[self.outputType],
                    self.batchSize, self.inputFieldShape, self.kernelShape,
                    self.inputChannelsPerConvGroup,
                    self.outputChannelsPerConvGroup, self.numConvGroups,
                    self.inputTransform, self.kernelTransform,
                    self.outputTransform))

    # -- the reference's member functions, answered by the C++ library ----
    def validate(self):
        _check(lib().mxconv_params_validate(byref(self.to_c())))

    def canonicalize(self):
        out = CParams()
        _check(lib().mxconv_params_canonicalize(byref(self.to_c()),
                                                byref(out)))
        return ConvParams.from_c(out)

    def getGradientParams(self):
        """poplin::getGradientParams(params), lib/poplin/ConvUtil.cpp:728-795."""
        out = CParams()
        _check(lib().mxconv_get_gradient_params(byref(self.to_c()), byref(out)))
        return ConvParams.from_c(out)

    def getWeightUpdateParams(self):
        """poplin::getWeightUpdateParams (lib/poplin/Convolution.cpp:3390)."""
        out = CParams()
        _check(lib().mxconv_get_weight_update_params(byref(self.to_c()),
                                                     byref(out)))
        return ConvParams.from_c(out)

    def _size(self, query, dim):
        v = c_uint64()
        _check(lib().mxconv_params_size(byref(self.to_c()), query, dim,
                                        byref(v)))
        return v.value

    def getTruncatedInputSize(self, dim):
        return self._size(0, dim)

    def getTruncatedKernelSize(self, dim):
        return self._size(1, dim)

    def getTransformedInputSize(self, dim):
        return self._size(2, dim)

    def getTransformedKernelSize(self, dim):
        return self._size(3, dim)

    def getUntransformedOutputSize(self, dim):
        return self._size(4, dim)

    def getOutputSize(self, dim):
        return self._size(5, dim)

    def getOutputFieldShape(self):
        return [self.getOutputSize(d)
                for d in range(len(self.inputFieldShape))]

    def getNumFieldDims(self):
        return len(self.inputFieldShape)

    def getNumInputChans(self):
        return self.inputChannelsPerConvGroup * self.numConvGroups

    def getNumOutputChans(self):
        return self.outputChannelsPerConvGroup * self.numConvGroups

    def isZeroConvolution(self):
        v = c_int()
        _check(lib().mxconv_params_is_zero_convolution(byref(self.to_c()),
                                                       byref(v)))
        return bool(v.value)

    def compare(self, other):
        v = c_int()
        _check(lib().mxconv_params_compare(byref(self.to_c()),
                                           byref(other.to_c()), byref(v)))
        return v.value

    def hash(self):
        v = c_uint64()
        _check(lib().mxconv_params_hash(byref(self.to_c()), byref(v)))
        return v.value

    def __str__(self):
        need = c_size_t()
        c = self.to_c()
        _check(lib().mxconv_params_to_string(byref(c), None, 0, byref(need)))
        buf = ctypes.create_string_buffer(need.value)
        _check(lib().mxconv_params_to_string(byref(c), buf, need.value,
                                             byref(need)))
        return buf.value.decode()

    # ConvUtil (include/poplin/ConvUtil.hpp)
    def getInputIndex(self, dim, outputIndex, kernelIndex):
        v = c_uint32()
        _check(lib().mxconv_get_input_index(byref(self.to_c()), dim,
                                            outputIndex, kernelIndex,
                                            byref(v)))
        return v.value

    def getKernelIndex(self, dim, outputIndex, inputIndex):
        v = c_uint32()
        _check(lib().mxconv_get_kernel_index(byref(self.to_c()), dim,
                                             outputIndex, inputIndex,
                                             byref(v)))
        return v.value

    def _range(self, query, dim, a, b):
        A = (c_uint32 * 2)(*a)
        B = (c_uint32 * 2)(*b)
        R = (c_uint32 * 2)()
        _check(lib().mxconv_get_range(byref(self.to_c()), query, dim, A, B, R))
        return (R[0], R[1])

    def getOutputRangeForKernelRange(self, dim, outputRange, kernelRange):
        return self._range(0, dim, outputRange, kernelRange)

    def getOutputRangeForKernelIndex(self, dim, outputRange, kernelIndex):
        return self._range(0, dim, outputRange, (kernelIndex, kernelIndex + 1))

    def getOutputRangeForInputRange(self, dim, outputRange, inputRange):
        return self._range(1, dim, outputRange, inputRange)

    def getOutputRangeForInputIndex(self, dim, outputRange, inputIndex):
        return self._range(1, dim, outputRange, (inputIndex, inputIndex + 1))

    def getInputRange(self, dim, outputRange, kernel):
        if isinstance(kernel, int):
            kernel = (kernel, kernel + 1)
        return self._range(2, dim, outputRange, kernel)

    def getKernelRange(self, dim, outputRange, inp):
        if isinstance(inp, int):
            inp = (inp, inp + 1)
        return self._range(3, dim, outputRange, inp)

    def getNumberOfMACs(self):
        v = c_uint64()
        _check(lib().mxconv_get_number_of_macs(byref(self.to_c()), byref(v)))
        return v.value

    def getFwdFlops(self):
        v = c_uint64()
        _check(lib().mxconv_get_fwd_flops(byref(self.to_c()), byref(v)))
        return v.value


def _option_arrays(options):
    options = options or {}
    keys = (c_char_p * max(len(options), 1))()
    values = (c_char_p * max(len(options), 1))()
    for i, (k, v) in enumerate(options.items()):
        keys[i] = str(k).encode()
        values[i] = str(v).encode()
    return keys, values, len(options)


def validate_options(options):
    """convolutionValidateOptions (include/poplin/Convolution.hpp:719)."""
    keys, values, n = _option_arrays(options)
    _check(lib().mxconv_validate_options(keys, values, n))


def quarter_metadata(fmt, scale):
    """Metadata byte of a quarter tensor: format 1 = E4M3, 0 = E5M2."""
    return ((fmt & 1) << 7) | (scale & 0x3f)


BUF_INPUT, BUF_WEIGHTS_PACKED, BUF_OUTPUT, BUF_BIAS, BUF_WORKSPACE, \
    BUF_WEIGHTS_EXTERNAL = range(6)


class Plan:
    """Owns an mxconv_plan.  Device pointers are plain integers (for torch
    tensors: `t.data_ptr()`); `stream` is a hipStream_t value or 0."""

    def __init__(self, params, options=None):
        self.params = params
        keys, values, n = _option_arrays(options)
        self._h = c_void_p()
        _check(lib().mxconv_plan_create(byref(params.to_c()), keys, values, n,
                                        byref(self._h)))

    def __del__(self):
        h = getattr(self, "_h", None)
        if h and _lib is not None:
            _lib.mxconv_plan_destroy(h)
            self._h = None

    def describe(self):
        need = c_size_t()
        _check(lib().mxconv_plan_describe(self._h, None, 0, byref(need)))
        buf = ctypes.create_string_buffer(need.value)
        _check(lib().mxconv_plan_describe(self._h, buf, need.value,
                                          byref(need)))
        return buf.value.decode()

    def constraints(self):
        """The plan as a complete planConstraints JSON document."""
        need = c_size_t()
        _check(lib().mxconv_plan_constraints(self._h, None, 0, byref(need)))
        buf = ctypes.create_string_buffer(need.value)
        _check(lib().mxconv_plan_constraints(self._h, buf, need.value,
                                             byref(need)))
        return buf.value.decode()

    COST_UNKNOWN = 2 ** 64 - 1

    def estimated_costs(self):
        """(cycles, memory bytes) the planner estimates for one launch:
        reportPlanEstimatedCosts (include/poplin/Convolution.hpp:590-611).
        cycles is COST_UNKNOWN where the cost model does not cover the
        kernel."""
        cycles, memory = c_uint64(), c_uint64()
        _check(lib().mxconv_plan_estimated_costs(self._h, byref(cycles),
                                                 byref(memory)))
        return cycles.value, memory.value

    def detailed_costs(self):
        """The estimate of estimated_costs taken apart: a dict with
        parallelSplit, serialSplit and (cycles, memory bytes) for
        rearrangement, compute, reduction and total:
        reportDetailedPlanEstimatedCosts
        (include/poplin/Convolution.hpp:613-676)."""
        c = DetailedCosts()
        _check(lib().mxconv_plan_detailed_costs(self._h, byref(c)))
        out = {"parallelSplit": c.parallel_split,
               "serialSplit": c.serial_split}
        for phase in ("rearrangement", "compute", "reduction", "total"):
            p = getattr(c, phase)
            out[phase] = (p.cycles, p.memory_bytes)
        return out

    def packs_like(self, other):
        """Whether weights packed for `other` are laid out as this plan
        reads them."""
        same = c_int32()
        _check(lib().mxconv_plans_pack_alike(self._h, other._h, byref(same)))
        return bool(same.value)

    def buffer_bytes(self, which):
        v = c_size_t()
        _check(lib().mxconv_plan_buffer_bytes(self._h, which, byref(v)))
        return v.value

    def pack_weights(self, weights_external, weights_packed, stream=0):
        _check(lib().mxconv_pack_weights(self._h, weights_external,
                                         weights_packed, stream))

    def acts_to_internal(self, external, internal, stream=0):
        _check(lib().mxconv_acts_to_internal(self._h, external, internal,
                                             stream))

    def acts_to_external(self, internal, external, stream=0):
        _check(lib().mxconv_acts_to_external(self._h, internal, external,
                                             stream))

    def fwd(self, inp, weights_packed, out, bias=None, workspace=None,
            workspace_bytes=0, stream=0):
        _check(lib().mxconv_fwd(self._h, inp, weights_packed, bias, out,
                                workspace, workspace_bytes, stream))

    def fwd_static_scratch(self, inp, weights_packed, out, bias=None,
                           stream=0):
        _check(lib().mxconv_fwd_static_scratch(self._h, inp, weights_packed,
                                               bias, out, stream))

    def fwd_quarter(self, inp, in_metadata, weights_packed, weights_metadata,
                    out, bias=None, workspace=None, workspace_bytes=0,
                    stream=0):
        _check(lib().mxconv_fwd_quarter(self._h, inp, in_metadata,
                                        weights_packed, weights_metadata, bias,
                                        out, workspace, workspace_bytes,
                                        stream))


def matMulParams(inputType, outputType, groups, m, k, n):
    """getConvParams of lib/poplin/MatMul.cpp:236-272: the convolution that
    computes C[g] = A[g] * B[g] for A [groups][m][k], B [groups][k][n]."""
    out = CParams()
    _check(lib().mxconv_matmul_params(inputType, outputType, groups, m, k, n,
                                      byref(out)))
    return ConvParams.from_c(out)


def matMulValidateOptions(options):
    """Checks matMul option keys and values (lib/poplin/MatMul.cpp:116-160)."""
    keys, values, n = _option_arrays(options)
    _check(lib().mxconv_matmul_validate_options(keys, values, n))


class MatMulPlan(Plan):
    """A plan for C[g] = A[g] * B[g], made from matMul options.  The operands
    are row-major device matrices A [groups][m][k], B [groups][k][n]; with one
    group A and C are the plan's input and output as they stand."""

    def __init__(self, inputType, outputType, groups, m, k, n, options=None):
        self.params = matMulParams(inputType, outputType, groups, m, k, n)
        self.groups, self.m, self.k, self.n = groups, m, k, n
        keys, values, num = _option_arrays(options)
        self._h = c_void_p()
        _check(lib().mxconv_matmul_plan_create(
            inputType, outputType, groups, m, k, n, keys, values, num,
            byref(self._h)))

    def pack_rhs(self, rhs, weights_packed, stream=0):
        _check(lib().mxconv_matmul_pack_rhs(self._h, rhs, weights_packed,
                                            stream))

    def lhs_to_internal(self, lhs, acts_internal, stream=0):
        _check(lib().mxconv_matmul_lhs_to_internal(self._h, lhs, acts_internal,
                                                   stream))

    def out_to_external(self, out_internal, result, stream=0):
        _check(lib().mxconv_matmul_out_to_external(self._h, out_internal,
                                                   result, stream))


class WeightUpdatePlan(Plan):
    """The plan of the weight update pass of the forward convolution
    ``fwd_params`` (poplin::calculateWeightDeltas /
    convolutionWeightUpdate).  Tensors are device pointers: z_deltas and
    activations channels-last, weights and weight deltas in the external
    [G][Co][Ci][kernel...] layout."""

    def __init__(self, fwd_params, options=None):
        self.fwd_params = fwd_params
        self.params = fwd_params.getWeightUpdateParams()
        keys, values, n = _option_arrays(options)
        self._h = c_void_p()
        _check(lib().mxconv_weight_update_plan_create(
            byref(fwd_params.to_c()), keys, values, n, byref(self._h)))

    def workspace_bytes(self):
        v = c_size_t()
        _check(lib().mxconv_weight_update_workspace_bytes(self._h, byref(v)))
        return v.value

    def calculate_weight_deltas(self, z_deltas, acts, weight_deltas, workspace,
                                workspace_bytes, stream=0):
        _check(lib().mxconv_calculate_weight_deltas(
            self._h, z_deltas, acts, weight_deltas, workspace, workspace_bytes,
            stream))

    def weight_update(self, z_deltas, weights, acts, scale, workspace,
                      workspace_bytes, stream=0):
        _check(lib().mxconv_convolution_weight_update(
            self._h, z_deltas, weights, acts, scale, workspace,
            workspace_bytes, stream))


def bias_update_workspace_bytes(outer_elems, channels):
    v = c_size_t()
    _check(lib().mxconv_bias_update_workspace_bytes(outer_elems, channels,
                                                    byref(v)))
    return v.value


def convolutionBiasUpdate(deltas_type, z_deltas, outer_elems, channels,
                          bias_type, biases, scale, workspace, workspace_bytes,
                          stream=0):
    """poplin::convolutionBiasUpdate on a channels-last z_deltas."""
    _check(lib().mxconv_convolution_bias_update(
        deltas_type, z_deltas, outer_elems, channels, bias_type, biases, scale,
        workspace, workspace_bytes, stream))


def multiconv_validate_options(options):
    """Checks multi-convolution options; True for planType parallel."""
    keys, values, n = _option_arrays(options)
    parallel = c_int(1)
    _check(lib().mxconv_multiconv_validate_options(keys, values, n,
                                                   byref(parallel)))
    return bool(parallel.value)


def multi_fwd(plans, inputs, weights_packed, outputs, biases=None,
              in_metadata=None, weights_metadata=None, workspaces=None,
              workspace_bytes=None, parallel=True, stream=0):
    """poplin::multiconv::convolution on device pointers: plans[i] run on
    (inputs[i], weights_packed[i]) into outputs[i]."""
    n = len(plans)

    def pointers(values):
        if values is None:
            return None
        return (c_void_p * max(n, 1))(*[v or None for v in values])

    def bytes_(values):
        if values is None:
            return None
        return (c_uint8 * max(n, 1))(*values)

    sizes = None
    if workspace_bytes is not None:
        sizes = (c_size_t * max(n, 1))(*workspace_bytes)
    _check(lib().mxconv_multi_fwd(
        n, pointers([p._h.value for p in plans]), pointers(inputs),
        bytes_(in_metadata), pointers(weights_packed),
        bytes_(weights_metadata), pointers(biases), pointers(outputs),
        pointers(workspaces), sizes, 1 if parallel else 0, stream))


def getWeightUpdateParams(params):
    """poplin::getWeightUpdateParams (lib/poplin/Convolution.cpp:3390-3435)."""
    return params.getWeightUpdateParams()


def getGradientParams(params):
    """poplin::getGradientParams (lib/poplin/ConvUtil.cpp:728-795)."""
    return params.getGradientParams()


def weightsTransposeChansFlipXY(params, weights_in, weights_out, stream=0):
    """poplin::weightsTransposeChansFlipXY on device pointers in the external
    layout; ``params`` are the forward parameters."""
    _check(lib().mxconv_weights_transpose_chans_flip_xy(
        byref(params.to_c()), weights_in, weights_out, stream))


def transposeGroupedMatrix(type_id, groups, rows, cols, src, dst, stream=0):
    """poplin::transposeGroupedMatrix as a device copy:
    src [groups][rows][cols] -> dst [groups][cols][rows]."""
    _check(lib().mxconv_transpose_grouped_matrix(type_id, groups, rows, cols,
                                                 src, dst, stream))


def scaled_add_to(type_id, c, scale_c, product, scale_product, elems,
                  stream=0):
    """c = scale_c * c + scale_product * product; poplin::matMulAcc is the
    case scale_c = 1."""
    _check(lib().mxconv_scaled_add_to(type_id, c, scale_c, product,
                                      scale_product, elems, stream))


def add_bias(type_id, acts, bias, outer_elems, channels, stream=0):
    _check(lib().mxconv_add_bias(type_id, acts, bias, outer_elems, channels,
                                 stream))

"""Python binding of the mxconv C ABI (include/mxconv.h).

This package is the ctypes stub a Python caller binds; all logic lives in
libmxconv.so (C++ host layer + HIP kernels for gfx950).  There is no CPU or
PyTorch fallback: importing works without a GPU (descriptor algebra and
planning are host code), any device call without the built library or without
a GPU raises.
"""
from .capi import (  # noqa: F401
    FLOAT, HALF, QUARTER, ConvParams, InputTransform, MatMulPlan, MxconvError,
    OutputTransform, Plan, Status, WeightUpdatePlan, add_bias,
    bias_update_workspace_bytes, build_library, convolutionBiasUpdate,
    getGradientParams, getWeightUpdateParams, lib, library_path, matMulParams,
    matMulValidateOptions, multi_fwd, multiconv_validate_options,
    quarter_metadata, scaled_add_to,
    transposeGroupedMatrix, validate_options, weightsTransposeChansFlipXY)

"""Loader for libTHCUNN.so - the role THCUNN.lua:7 (`ffi.load('libTHCUNN')`) plays
for LuaJIT. The library is built in-tree by ``__graft_entry__.build()`` /
``make -C cunn_amd/csrc``; there is no fallback: without it every call fails."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libTHCUNN.so")

# The 14 fp32 entry points of the hot path (include/THCUNN.h).
ENTRY_POINTS = [
    "BatchNormalization_updateOutput", "BatchNormalization_backward",
    "SpatialAveragePooling_updateOutput", "SpatialAveragePooling_updateGradInput",
    "SpatialConvolutionMM_updateOutput", "SpatialConvolutionMM_updateGradInput",
    "SpatialConvolutionMM_accGradParameters",
    "SpatialDepthWiseConvolution_updateOutput", "SpatialDepthWiseConvolution_updateGradInput",
    "SpatialDepthWiseConvolution_accGradParameters",
    "SpatialDilatedMaxPooling_updateOutput", "SpatialDilatedMaxPooling_updateGradInput",
    "SpatialMaxPooling_updateOutput", "SpatialMaxPooling_updateGradInput",
    "SpatialDilatedConvolution_updateOutput", "SpatialDilatedConvolution_updateGradInput",
    "SpatialDilatedConvolution_accGradParameters",
    "SpatialFullDilatedConvolution_updateOutput", "SpatialFullDilatedConvolution_updateGradInput",
    "SpatialFullDilatedConvolution_accGradParameters",
    "SpatialFullConvolution_updateOutput", "SpatialFullConvolution_updateGradInput",
    "SpatialFullConvolution_accGradParameters",
    "Threshold_updateOutput", "Threshold_updateGradInput",
    # no counterpart in the reference: for callers that cannot allocate device memory
    "SpatialDepthWiseConvolution_accGradParameters_noAlloc",
    # no counterpart in the reference: BatchNormalization + Threshold(0, 0) in one pass (include/THCUNN_fused.h)
    "BatchNormalizationReLU_updateOutput", "BatchNormalizationReLU_backward",
    # no counterpart in the reference: SpatialConvolutionMM + Threshold(0, 0) in one pass (include/THCUNN_fused.h)
    "SpatialConvolutionMMReLU_updateOutput",
]

_T = C.c_void_p  # THCudaTensor* / THCudaLongTensor* / THCState*
_i, _b, _f, _d = C.c_int, C.c_bool, C.c_float, C.c_double

SIGNATURES = {
    "BatchNormalization_updateOutput": [_T] * 9 + [_b, _d, _d],
    "BatchNormalization_backward": [_T] * 11 + [_b, _d, _d],
    "SpatialAveragePooling_updateOutput": [_T] * 3 + [_i] * 6 + [_b, _b],
    "SpatialAveragePooling_updateGradInput": [_T] * 4 + [_i] * 6 + [_b, _b],
    "SpatialConvolutionMM_updateOutput": [_T] * 7 + [_i] * 6,
    "SpatialConvolutionMM_updateGradInput": [_T] * 7 + [_i] * 6,
    "SpatialConvolutionMM_accGradParameters": [_T] * 7 + [_i] * 6 + [_f],
    "SpatialDepthWiseConvolution_updateOutput": [_T] * 7 + [_i] * 6,
    "SpatialDepthWiseConvolution_updateGradInput": [_T] * 7 + [_i] * 6,
    "SpatialDepthWiseConvolution_accGradParameters": [_T] * 7 + [_i] * 6 + [_f],
    "SpatialDilatedMaxPooling_updateOutput": [_T] * 4 + [_i] * 8 + [_b],
    "SpatialDilatedMaxPooling_updateGradInput": [_T] * 5 + [_i] * 8 + [_b],
    "SpatialMaxPooling_updateOutput": [_T] * 4 + [_i] * 6 + [_b],
    "SpatialMaxPooling_updateGradInput": [_T] * 5 + [_i] * 6 + [_b],
    "SpatialDilatedConvolution_updateOutput": [_T] * 7 + [_i] * 8,
    "SpatialDilatedConvolution_updateGradInput": [_T] * 6 + [_i] * 8,
    "SpatialDilatedConvolution_accGradParameters": [_T] * 7 + [_i] * 8 + [_f],
    "SpatialFullDilatedConvolution_updateOutput": [_T] * 7 + [_i] * 10,
    "SpatialFullDilatedConvolution_updateGradInput": [_T] * 6 + [_i] * 10,
    "SpatialFullDilatedConvolution_accGradParameters": [_T] * 7 + [_i] * 10 + [_f],
    "SpatialFullConvolution_updateOutput": [_T] * 7 + [_i] * 8,
    "SpatialFullConvolution_updateGradInput": [_T] * 6 + [_i] * 8,
    "SpatialFullConvolution_accGradParameters": [_T] * 7 + [_i] * 8 + [_f],
    "Threshold_updateOutput": [_T] * 3 + [_f, _f, _b],
    "Threshold_updateGradInput": [_T] * 4 + [_f, _f, _b],
    "SpatialDepthWiseConvolution_accGradParameters_noAlloc": [_T] * 5 + [_i] * 6 + [_f],
    "BatchNormalizationReLU_updateOutput": [_T] * 9 + [_b, _d, _d],
    "BatchNormalizationReLU_backward": [_T] * 12 + [_b, _d, _d],
    "SpatialConvolutionMMReLU_updateOutput": [_T] * 7 + [_i] * 6,
}

_LP = C.POINTER(C.c_long)
SHIM = {  # name: (restype, argtypes)
    "THCState_alloc": (_T, []),
    "THCState_free": (None, [_T]),
    "THCState_setCurrentStream": (None, [_T, _T]),
    "THCState_getCurrentStream": (_T, [_T]),
    "THCState_synchronize": (None, [_T]),
    "THSetErrorHandler": (None, [_T, _T]),
    "THSetArgErrorHandler": (None, [_T, _T]),
    "THCudaTensor_new": (_T, [_T]),
    "THCudaTensor_newWithSize": (_T, [_T, _i, _LP]),
    "THCudaTensor_newWithData": (_T, [_T, _T, C.c_ssize_t, C.c_ssize_t, _i, _LP, _LP]),
    "THCudaTensor_newView": (_T, [_T, _T, C.c_ssize_t, _i, _LP, _LP]),
    "THCudaTensor_retain": (None, [_T, _T]),
    "THCudaTensor_free": (None, [_T, _T]),
    "THCudaTensor_resizeNd": (None, [_T, _T, _i, _LP]),
    "THCudaTensor_data": (_T, [_T, _T]),
    "THCudaTensor_nDimension": (_i, [_T, _T]),
    "THCudaTensor_size": (C.c_long, [_T, _T, _i]),
    "THCudaTensor_stride": (C.c_long, [_T, _T, _i]),
    "THCudaTensor_nElement": (C.c_ssize_t, [_T, _T]),
    "THCudaTensor_isContiguous": (_i, [_T, _T]),
    "THCudaTensor_fill": (None, [_T, _T, _f]),
    "THCudaTensor_copy": (None, [_T, _T, _T]),
    "THCudaTensor_copyFromHost": (None, [_T, _T, _T]),
    "THCudaTensor_copyToHost": (None, [_T, _T, _T]),
    "THCudaLongTensor_new": (_T, [_T]),
    "THCudaLongTensor_newWithSize": (_T, [_T, _i, _LP]),
    "THCudaLongTensor_newWithData": (_T, [_T, _T, C.c_ssize_t, C.c_ssize_t, _i, _LP, _LP]),
    "THCudaLongTensor_free": (None, [_T, _T]),
    "THCudaLongTensor_resizeNd": (None, [_T, _T, _i, _LP]),
    "THCudaLongTensor_data": (_T, [_T, _T]),
    "THCudaLongTensor_nDimension": (_i, [_T, _T]),
    "THCudaLongTensor_size": (C.c_long, [_T, _T, _i]),
    "THCudaLongTensor_nElement": (C.c_ssize_t, [_T, _T]),
    "THCudaLongTensor_copyFromHost": (None, [_T, _T, _T]),
    "THCudaLongTensor_copyToHost": (None, [_T, _T, _T]),
    "THCUNN_setSwitch": (_i, [C.c_char_p, C.c_char_p]),
    "THNN_Cuda_im2col": (None, [_T, _T] + [_i] * 12 + [_T]),
    "THNN_Cuda_col2im": (None, [_T, _T] + [_i] * 12 + [_T]),
}

_lib = None


def load() -> C.CDLL:
    """dlopen the library and type every exported symbol. Raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C cunn_amd/csrc` (there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, "THNN_Cuda" + name)
        fn.restype = None
        fn.argtypes = args
    for name, (res, args) in SHIM.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib

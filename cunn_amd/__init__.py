"""MI355X-native THCUNN spatial-convolution hot path.

`cunn_amd.THNN` mirrors what ``THCUNN.lua`` builds for ``torch.CudaTensor``: a
table of functions named like the reference's (``SpatialDepthWiseConvolution_updateOutput``
...) that prepend the THCState and call the ``THNN_Cuda*`` symbol of
``libTHCUNN.so``. `set_switch` forces one of the kernel families that compute the
same results (what the parity tests use).
"""
from . import _lib
from .tensor import CudaTensor, CudaLongTensor, THError, state, synchronize
from .thnn import THNN


def set_switch(name, value):
    """THCUNN_setSwitch: force a kernel family (``value`` as the environment variable of the same name
    would hold it, ``None`` = the default choice by shape)."""
    ok = _lib.load().THCUNN_setSwitch(name.encode(), None if value is None else str(value).encode())
    if not ok:
        raise KeyError(name)


__all__ = ["CudaTensor", "CudaLongTensor", "THError", "THNN", "state", "synchronize", "set_switch", "_lib"]

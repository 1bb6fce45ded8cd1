"""MI355X-native THCUNN spatial-convolution hot path.

`cunn_amd.THNN` mirrors what ``THCUNN.lua`` builds for ``torch.CudaTensor``: a
table of functions named like the reference's (``SpatialDepthWiseConvolution_updateOutput``
...) that prepend the THCState and call the ``THNN_Cuda*`` symbol of
``libTHCUNN.so``. `cunn_amd.nn` mirrors the torch/nn modules that own the
buffers those functions take.
"""
from . import _lib
from .tensor import CudaTensor, CudaLongTensor, THError, state, synchronize
from .thnn import THNN

__all__ = ["CudaTensor", "CudaLongTensor", "THError", "THNN", "state", "synchronize", "_lib"]

"""ctypes front end of the CPU oracle (``thnn_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the shipped package never imports
it. Functions take and return NumPy arrays laid out as the THNN entry points see
their tensors (fp32 NCHW, int64 1-based max-pool indices) and mirror the
argument order of lib/THCUNN/generic/THCUNN.h (kW, kH, dW, dH, padW, padH).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libthnn_oracle.so")


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "thnn_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libthnn_oracle.so"])
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        _lib.oracle_num_threads.restype = C.c_int
        _lib.oracle_pool_out_size_fixed.restype = C.c_int
    return _lib


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    if a is None:
        return C.c_void_p(None)
    return a.ctypes.data_as(C.c_void_p)


def conv_out_size(n, k, d, pad, dil=1):
    return (n + 2 * pad - (dil * (k - 1) + 1)) // d + 1


def pool_out_size(n, k, d, pad, dil, ceil_mode, any_pad):
    return int(lib().oracle_pool_out_size_fixed(int(n), int(k), int(d), int(pad), int(dil),
                                                int(bool(ceil_mode)), int(bool(any_pad))))


# ---------------------------------------------------------------- im2col ----
def im2col(im, kW, kH, dW, dH, padW, padH, dilW=1, dilH=1):
    im = _f(im)
    Cc, H, W = im.shape
    oH, oW = conv_out_size(H, kH, dH, padH, dilH), conv_out_size(W, kW, dW, padW, dilW)
    col = np.empty((Cc * kH * kW, oH * oW), np.float32)
    lib().oracle_im2col(_p(im), Cc, H, W, kH, kW, padH, padW, dH, dW, dilH, dilW, _p(col))
    return col


def col2im(col, Cc, H, W, kW, kH, dW, dH, padW, padH, dilW=1, dilH=1):
    col = _f(col)
    oH, oW = conv_out_size(H, kH, dH, padH, dilH), conv_out_size(W, kW, dW, padW, dilW)
    assert col.shape == (Cc * kH * kW, oH * oW)
    im = np.empty((Cc, H, W), np.float32)
    lib().oracle_col2im(_p(col), Cc, H, W, oH, oW, kH, kW, padH, padW, dH, dW, dilH, dilW, _p(im))
    return im


# ------------------------------------------------------------- depthwise ----
def dwconv_updateOutput(x, weight, bias, kW, kH, dW, dH, padW, padH):
    x, weight = _f(x), _f(weight)
    N, Cc, H, W = x.shape
    M = weight.shape[0]
    assert weight.shape == (M, Cc, kH, kW)
    bias = None if bias is None else _f(bias)
    oH, oW = conv_out_size(H, kH, dH, padH), conv_out_size(W, kW, dW, padW)
    out = np.empty((N, Cc * M, oH, oW), np.float32)
    lib().oracle_dwconv_updateOutput(_p(x), _p(weight), _p(bias), _p(out), N, Cc, M, H, W,
                                     kW, kH, dW, dH, padW, padH)
    return out


def dwconv_updateGradInput(x_shape, gradOut, weight, kW, kH, dW, dH, padW, padH):
    gradOut, weight = _f(gradOut), _f(weight)
    N, Cc, H, W = x_shape
    M = weight.shape[0]
    gi = np.empty((N, Cc, H, W), np.float32)
    lib().oracle_dwconv_updateGradInput(_p(gradOut), _p(weight), _p(gi), N, Cc, M, H, W,
                                        kW, kH, dW, dH, padW, padH)
    return gi


def dwconv_accGradParameters(x, gradOut, gradWeight, gradBias, kW, kH, dW, dH, padW, padH, scale=1.0):
    """gradWeight (M,C,kH,kW) / gradBias (M,C) are accumulated into in place and returned."""
    x, gradOut = _f(x), _f(gradOut)
    N, Cc, H, W = x.shape
    M = gradWeight.shape[0]
    assert gradWeight.dtype == np.float32 and gradWeight.flags.c_contiguous
    if gradBias is not None:
        assert gradBias.dtype == np.float32 and gradBias.flags.c_contiguous
    lib().oracle_dwconv_accGradParameters(_p(x), _p(gradOut), _p(gradWeight), _p(gradBias), N, Cc, M,
                                          H, W, kW, kH, dW, dH, padW, padH, C.c_float(scale))
    return gradWeight, gradBias


# ---------------------------------------------------------------- ConvMM ----
def convmm_updateOutput(x, weight, bias, kW, kH, dW, dH, padW, padH):
    x = _f(x)
    N, Cin, H, W = x.shape
    weight = _f(weight).reshape(weight.shape[0], -1)
    Cout = weight.shape[0]
    assert weight.shape[1] == Cin * kH * kW
    bias = None if bias is None else _f(bias)
    oH, oW = conv_out_size(H, kH, dH, padH), conv_out_size(W, kW, dW, padW)
    out = np.empty((N, Cout, oH, oW), np.float32)
    lib().oracle_convmm_updateOutput(_p(x), _p(weight), _p(bias), _p(out), N, Cin, Cout, H, W,
                                     kW, kH, dW, dH, padW, padH)
    return out


def convmm_updateGradInput(x_shape, gradOut, weight, kW, kH, dW, dH, padW, padH):
    gradOut = _f(gradOut)
    N, Cin, H, W = x_shape
    weight = _f(weight).reshape(weight.shape[0], -1)
    Cout = weight.shape[0]
    gi = np.empty((N, Cin, H, W), np.float32)
    lib().oracle_convmm_updateGradInput(_p(gradOut), _p(weight), _p(gi), N, Cin, Cout, H, W,
                                        kW, kH, dW, dH, padW, padH)
    return gi


def convmm_accGradParameters(x, gradOut, gradWeight, gradBias, kW, kH, dW, dH, padW, padH, scale=1.0):
    x, gradOut = _f(x), _f(gradOut)
    N, Cin, H, W = x.shape
    Cout = gradWeight.shape[0]
    assert gradWeight.dtype == np.float32 and gradWeight.flags.c_contiguous
    lib().oracle_convmm_accGradParameters(_p(x), _p(gradOut), _p(gradWeight), _p(gradBias), N, Cin,
                                          Cout, H, W, kW, kH, dW, dH, padW, padH, C.c_float(scale))
    return gradWeight, gradBias


# ------------------------------------------------- dilated convolution ----
def dilconv_updateOutput(x, weight, bias, kW, kH, dW, dH, padW, padH, dilW, dilH):
    x = _f(x)
    N, Cin, H, W = x.shape
    weight = _f(weight).reshape(weight.shape[0], -1)
    Cout = weight.shape[0]
    assert weight.shape[1] == Cin * kH * kW
    bias = None if bias is None else _f(bias)
    oH, oW = conv_out_size(H, kH, dH, padH, dilH), conv_out_size(W, kW, dW, padW, dilW)
    out = np.empty((N, Cout, oH, oW), np.float32)
    lib().oracle_dilconv_updateOutput(_p(x), _p(weight), _p(bias), _p(out), N, Cin, Cout, H, W,
                                      kW, kH, dW, dH, padW, padH, dilW, dilH)
    return out


def dilconv_updateGradInput(x_shape, gradOut, weight, kW, kH, dW, dH, padW, padH, dilW, dilH):
    gradOut = _f(gradOut)
    N, Cin, H, W = x_shape
    weight = _f(weight).reshape(weight.shape[0], -1)
    gi = np.empty((N, Cin, H, W), np.float32)
    lib().oracle_dilconv_updateGradInput(_p(gradOut), _p(weight), _p(gi), N, Cin, weight.shape[0], H, W,
                                         kW, kH, dW, dH, padW, padH, dilW, dilH)
    return gi


def dilconv_accGradParameters(x, gradOut, gradWeight, gradBias, kW, kH, dW, dH, padW, padH, dilW, dilH, scale=1.0):
    x, gradOut = _f(x), _f(gradOut)
    N, Cin, H, W = x.shape
    assert gradWeight.dtype == np.float32 and gradWeight.flags.c_contiguous
    lib().oracle_dilconv_accGradParameters(_p(x), _p(gradOut), _p(gradWeight), _p(gradBias), N, Cin,
                                           gradWeight.shape[0], H, W, kW, kH, dW, dH, padW, padH, dilW, dilH,
                                           C.c_float(scale))
    return gradWeight, gradBias


# ---------------------------------------------- transposed convolution ----
def full_out_size(n, k, d, pad, dil, adj):
    return (n - 1) * d - 2 * pad + (dil * (k - 1) + 1) + adj


def fullconv_updateOutput(x, weight, bias, kW, kH, dW, dH, padW, padH, dilW=1, dilH=1, adjW=0, adjH=0):
    """weight (Cin, Cout, kH, kW)"""
    x, weight = _f(x), _f(weight)
    N, Cin, H, W = x.shape
    Cout = weight.shape[1]
    assert weight.shape == (Cin, Cout, kH, kW)
    bias = None if bias is None else _f(bias)
    oH, oW = full_out_size(H, kH, dH, padH, dilH, adjH), full_out_size(W, kW, dW, padW, dilW, adjW)
    out = np.empty((N, Cout, oH, oW), np.float32)
    lib().oracle_fullconv_updateOutput(_p(x), _p(weight), _p(bias), _p(out), N, Cin, Cout, H, W, oH, oW,
                                       kW, kH, dW, dH, padW, padH, dilW, dilH)
    return out


def _full_check(H, W, oH, oW, kW, kH, dW, dH, padW, padH, dilW, dilH):
    # The reference's im2col over the output-sized image produces conv_out(oH) x conv_out(oW) columns and
    # assumes that this is H x W (generic/SpatialFullDilatedConvolution.cu:255, 268-273); with an output
    # padding >= stride (allowed when it is < dilation) that does not hold and the reference overruns its buffer.
    if conv_out_size(oH, kH, dH, padH, dilH) != H or conv_out_size(oW, kW, dW, padW, dilW) != W:
        raise ValueError("output padding >= stride: not defined by the reference's backward passes")


def fullconv_updateGradInput(x_shape, gradOut, weight, kW, kH, dW, dH, padW, padH, dilW=1, dilH=1, adjW=0, adjH=0):
    gradOut, weight = _f(gradOut), _f(weight)
    N, Cin, H, W = x_shape
    Cout = weight.shape[1]
    oH, oW = gradOut.shape[2:]
    _full_check(H, W, oH, oW, kW, kH, dW, dH, padW, padH, dilW, dilH)
    gi = np.empty((N, Cin, H, W), np.float32)
    lib().oracle_fullconv_updateGradInput(_p(gradOut), _p(weight), _p(gi), N, Cin, Cout, H, W, oH, oW,
                                          kW, kH, dW, dH, padW, padH, dilW, dilH)
    return gi


def fullconv_accGradParameters(x, gradOut, gradWeight, gradBias, kW, kH, dW, dH, padW, padH, dilW=1, dilH=1,
                               adjW=0, adjH=0, scale=1.0):
    x, gradOut = _f(x), _f(gradOut)
    N, Cin, H, W = x.shape
    Cout = gradWeight.shape[1]
    oH, oW = gradOut.shape[2:]
    _full_check(H, W, oH, oW, kW, kH, dW, dH, padW, padH, dilW, dilH)
    assert gradWeight.dtype == np.float32 and gradWeight.flags.c_contiguous
    lib().oracle_fullconv_accGradParameters(_p(x), _p(gradOut), _p(gradWeight), _p(gradBias), N, Cin, Cout,
                                            H, W, oH, oW, kW, kH, dW, dH, padW, padH, dilW, dilH, C.c_float(scale))
    return gradWeight, gradBias


# -------------------------------------------------------------------- BN ----
def _ncl(x):
    x = _f(x)
    N, Cc = x.shape[0], x.shape[1]
    L = int(np.prod(x.shape[2:])) if x.ndim > 2 else 1
    return x, N, Cc, L


def bn_updateOutput(x, weight, bias, runningMean, runningVar, train, momentum, eps):
    """Returns (output, saveMean, saveStd); runningMean/runningVar are updated in place."""
    x, N, Cc, L = _ncl(x)
    out = np.empty_like(x)
    saveMean = np.zeros(Cc, np.float32)
    saveStd = np.zeros(Cc, np.float32)
    weight = None if weight is None else _f(weight)
    bias = None if bias is None else _f(bias)
    assert runningMean.dtype == np.float32 and runningVar.dtype == np.float32
    lib().oracle_bn_updateOutput(_p(x), _p(out), _p(weight), _p(bias), _p(runningMean), _p(runningVar),
                                 _p(saveMean), _p(saveStd), N, Cc, L, int(bool(train)),
                                 C.c_double(momentum), C.c_double(eps))
    return out, saveMean, saveStd


def bn_backward(x, gradOut, weight, runningMean, runningVar, saveMean, saveStd, train, scale, eps,
                gradWeight=None, gradBias=None, want_gradInput=True):
    """gradWeight/gradBias (float32 arrays or None) are accumulated into in place."""
    x, N, Cc, L = _ncl(x)
    gradOut = _f(gradOut)
    gi = np.empty_like(x) if want_gradInput else None
    weight = None if weight is None else _f(weight)
    lib().oracle_bn_backward(_p(x), _p(gradOut), _p(gi), _p(gradWeight), _p(gradBias), _p(weight),
                             _p(_f(runningMean)), _p(_f(runningVar)), _p(_f(saveMean)), _p(_f(saveStd)),
                             N, Cc, L, int(bool(train)), C.c_double(scale), C.c_double(eps))
    return gi, gradWeight, gradBias


# --------------------------------------------------------------- pooling ----
def maxpool_updateOutput(x, kW, kH, dW, dH, padW, padH, ceil_mode, dilW=1, dilH=1):
    x = _f(x)
    N, Cc, H, W = x.shape
    anyp = bool(padW or padH)
    oH = pool_out_size(H, kH, dH, padH, dilH, ceil_mode, anyp)
    oW = pool_out_size(W, kW, dW, padW, dilW, ceil_mode, anyp)
    out = np.empty((N, Cc, oH, oW), np.float32)
    idx = np.empty((N, Cc, oH, oW), np.int64)
    lib().oracle_maxpool_updateOutput(_p(x), _p(out), _p(idx), N, Cc, H, W, oH, oW, kW, kH, dW, dH,
                                      padW, padH, dilW, dilH)
    return out, idx


def maxpool_updateGradInput(x_shape, gradOut, indices, kW, kH, dW, dH, padW, padH, ceil_mode, dilW=1, dilH=1):
    gradOut = _f(gradOut)
    indices = np.ascontiguousarray(indices, dtype=np.int64)
    N, Cc, H, W = x_shape
    oH, oW = gradOut.shape[2:]
    gi = np.empty((N, Cc, H, W), np.float32)
    lib().oracle_maxpool_updateGradInput(_p(gradOut), _p(indices), _p(gi), N, Cc, H, W, oH, oW, kW, kH,
                                         dW, dH, padW, padH, dilW, dilH)
    return gi


def avgpool_updateOutput(x, kW, kH, dW, dH, padW, padH, ceil_mode, count_include_pad):
    x = _f(x)
    N, Cc, H, W = x.shape
    anyp = bool(padW or padH)
    oH = pool_out_size(H, kH, dH, padH, 1, ceil_mode, anyp)
    oW = pool_out_size(W, kW, dW, padW, 1, ceil_mode, anyp)
    out = np.empty((N, Cc, oH, oW), np.float32)
    lib().oracle_avgpool_updateOutput(_p(x), _p(out), N, Cc, H, W, oH, oW, kW, kH, dW, dH, padW, padH,
                                      int(bool(count_include_pad)))
    return out


def avgpool_updateGradInput(x_shape, gradOut, kW, kH, dW, dH, padW, padH, ceil_mode, count_include_pad):
    gradOut = _f(gradOut)
    N, Cc, H, W = x_shape
    oH, oW = gradOut.shape[2:]
    gi = np.empty((N, Cc, H, W), np.float32)
    lib().oracle_avgpool_updateGradInput(_p(gradOut), _p(gi), N, Cc, H, W, oH, oW, kW, kH, dW, dH,
                                         padW, padH, int(bool(count_include_pad)))
    return gi


# ------------------------------------------------------------- Threshold ----
def threshold_updateOutput(x, threshold, val):
    """lib/THCUNN/Threshold.cu:6-22: out = x > threshold ? x : val (a NaN input gives val)."""
    x = _f(x)
    return np.where(x > np.float32(threshold), x, np.float32(val)).astype(np.float32)


def threshold_updateGradInput(x, gradOut, threshold):
    """lib/THCUNN/Threshold.cu:42-56: gradIn = x > threshold ? gradOut : 0."""
    x, gradOut = _f(x), _f(gradOut)
    return np.where(x > np.float32(threshold), gradOut.reshape(x.shape), np.float32(0)).astype(np.float32)

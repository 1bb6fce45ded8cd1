"""GPU parity of SpatialDilatedConvolution and SpatialFull(Dilated)Convolution through the C ABI
against the CPU oracle (same tolerances as SpatialConvolutionMM: 1e-5 rel / 1e-4 abs outputs and
gradients, 1e-3 rel weight gradients). The cases cover every kernel path: zero-bordered fast
kernels (K % 16 == 0), generic kernels, stride-1 gradInput through the forward kernel, gradient
columns + col2im, output padding, 3-D inputs, non-contiguous inputs, accumulation with scale."""
import os

import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402
from test_gpu_parity import T, close, WG_RTOL, WG_ATOL  # noqa: E402,F401

DIL_CASES = [
    # N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH
    (4, 16, 32, 28, 28, 3, 3, 1, 1, 2, 2, 2, 2),     # "same" dilated 3x3, fast kernels, stride-1 gradInput
    (3, 8, 24, 21, 25, 3, 3, 1, 1, 0, 0, 3, 2),      # no padding, dilated, K % 16 != 0 -> generic forward
    (2, 16, 16, 30, 30, 3, 3, 2, 2, 1, 1, 2, 2),     # stride 2: gradient columns + col2im
    (2, 5, 7, 19, 23, 2, 4, 1, 2, 1, 3, 4, 1),       # rectangular everything
    (2, 32, 8, 16, 16, 1, 1, 1, 1, 0, 0, 5, 5),      # 1x1: dilation without effect
    (2, 16, 16, 20, 20, 3, 3, 1, 1, 5, 5, 2, 2),     # pad > dil*(k-1): gradInput cannot use the forward kernel
    (5, 16, 8, 40, 44, 5, 5, 1, 1, 4, 4, 2, 2),      # L % 16 != 0 in the weight-gradient kernel
]


def _dil_run(T, case, bias=True, xt=None, scale=1.0, seed=80, single=False):
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH = case
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(seed)
    K = Cin * kH * kW
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kH, kW)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32) if bias else None
    args = (kW, kH, dW, dH, pW, pH, dlW, dlH)
    xin = x[0] if single else x
    tx = xt(xin) if xt else CT.from_numpy(xin)
    tw, tb = CT.from_numpy(w), (CT.from_numpy(b) if bias else None)
    out, cols, ones = CT(), CT(), CT()
    THNN.SpatialDilatedConvolution_updateOutput(tx, out, tw, tb, cols, ones, *args)
    ry = O.dilconv_updateOutput(x, w, b, *args)
    y = out.numpy()
    assert y.shape == (ry[0].shape if single else ry.shape)
    close(y, ry[0] if single else ry)
    gy = rng.standard_normal(ry.shape).astype(np.float32)
    tgy = CT.from_numpy(gy[0] if single else gy)
    gi = CT()
    THNN.SpatialDilatedConvolution_updateGradInput(tx, tgy, gi, tw, CT(), *args)
    rgi = O.dilconv_updateGradInput(x.shape, gy, w, *args)
    close(gi.numpy(), rgi[0] if single else rgi)
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    tgw, tgb = CT.from_numpy(gw0), (CT.from_numpy(gb0) if bias else None)
    THNN.SpatialDilatedConvolution_accGradParameters(tx, tgy, tgw, tgb, cols, ones, *args, scale)
    rgw, rgb = O.dilconv_accGradParameters(x, gy, gw0.reshape(Cout, K).copy(), gb0.copy() if bias else None, *args,
                                           scale=scale)
    close(tgw.numpy().reshape(Cout, K), rgw, WG_RTOL, WG_ATOL * max(1.0, abs(scale)) * 4)
    if bias:
        close(tgb.numpy(), rgb, WG_RTOL, WG_ATOL * max(1.0, abs(scale)) * 4)


def _offset_tensor(T, a, off):
    """A contiguous tensor whose first element sits `off` floats behind a 16-byte boundary of its storage."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    big = T.CudaTensor.with_size(a.size + 8)
    big.fill(float("nan"))
    strides = [1] * a.ndim
    for d in range(a.ndim - 2, -1, -1):
        strides[d] = strides[d + 1] * a.shape[d + 1]
    v = big.view(off, a.shape, strides)
    v.copy_(a)
    return v


@pytest.mark.parametrize("case,off", [
    ((3, 8, 20, 9, 9, 3, 3, 1, 1, 1, 1), 0),      # 81 positions per image: rows padded to 84
    ((2, 16, 24, 7, 7, 1, 1, 1, 1, 0, 0), 0),     # 1x1 at 7x7: padded rows, images read in place
    ((2, 8, 20, 8, 8, 3, 3, 1, 1, 1, 1), 1),      # rows of 64 floats that start off a 16-byte boundary
    ((2, 5, 12, 13, 11, 3, 3, 2, 2, 1, 1), 3),    # stride 2, 42 positions, odd offset
])
def test_weight_gradient_with_unaligned_gradoutput_rows(T, case, off):
    """gradOutput rows that are not whole 16-byte groups (length not a multiple of 4, or the tensor starts off a
    16-byte boundary) are copied into zero-padded rows first; the padding must not reach any sum."""
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH = case
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(90 + off)
    K = Cin * kH * kW
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    oH, oW = (H + 2 * pH - kH) // dH + 1, (W + 2 * pW - kW) // dW + 1
    gy = rng.standard_normal((N, Cout, oH, oW)).astype(np.float32)
    gw0 = rng.standard_normal((Cout, K)).astype(np.float32)
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    tgw, tgb = CT.from_numpy(gw0), CT.from_numpy(gb0)
    tgy = _offset_tensor(T, gy, off) if off else CT.from_numpy(gy)
    THNN.SpatialConvolutionMM_accGradParameters(CT.from_numpy(x), tgy, tgw, tgb, CT(), CT(), kW, kH, dW, dH, pW, pH, 0.5)
    rgw, rgb = O.dilconv_accGradParameters(x, gy, gw0.copy(), gb0.copy(), kW, kH, dW, dH, pW, pH, 1, 1, scale=0.5)
    close(tgw.numpy(), rgw, WG_RTOL, WG_ATOL * 4)
    close(tgb.numpy(), rgb, WG_RTOL, WG_ATOL * 4)


@pytest.mark.parametrize("case", DIL_CASES)
def test_dilated_convolution(T, case):
    _dil_run(T, case)


def test_dilated_convolution_variants(T):
    rng = np.random.default_rng(81)
    _dil_run(T, DIL_CASES[0], bias=False, scale=0.5)
    _dil_run(T, DIL_CASES[3], xt=lambda a: T.CudaTensor.noncontiguous_from_numpy(a, rng), scale=2.0)
    _dil_run(T, (1,) + DIL_CASES[1][1:], single=True)
    cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", "1")
    try:
        _dil_run(T, DIL_CASES[0])
        _dil_run(T, DIL_CASES[2])
    finally:
        cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", None)


def test_dilated_convolution_dilation_one_is_convmm(T):
    """With dilation 1 the entry point gives bit-identical results to SpatialConvolutionMM."""
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(82)
    x = rng.standard_normal((3, 16, 20, 24)).astype(np.float32)
    w = (rng.standard_normal((8, 16, 3, 3)) * 0.1).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    a, c = CT(), CT()
    THNN.SpatialDilatedConvolution_updateOutput(CT.from_numpy(x), a, CT.from_numpy(w), CT.from_numpy(b), CT(), CT(),
                                                3, 3, 1, 1, 1, 1, 1, 1)
    THNN.SpatialConvolutionMM_updateOutput(CT.from_numpy(x), c, CT.from_numpy(w), CT.from_numpy(b), CT(), CT(),
                                           3, 3, 1, 1, 1, 1)
    assert np.array_equal(a.numpy(), c.numpy())


def test_dilated_convolution_errors(T):
    THNN, CT = T.THNN, T.CudaTensor
    x = CT.from_numpy(np.zeros((1, 4, 8, 8), np.float32))
    w2 = CT.from_numpy(np.zeros((4, 36), np.float32))
    w4 = CT.from_numpy(np.zeros((4, 4, 3, 3), np.float32))
    with pytest.raises(T.THError, match="4D weight tensor"):
        THNN.SpatialDilatedConvolution_updateOutput(x, CT(), w2, None, CT(), CT(), 3, 3, 1, 1, 0, 0, 1, 1)
    with pytest.raises(T.THError, match="dilation should be greater than 0"):
        THNN.SpatialDilatedConvolution_updateOutput(x, CT(), w4, None, CT(), CT(), 3, 3, 1, 1, 0, 0, 0, 1)
    with pytest.raises(T.THError, match="Output size is too small"):
        THNN.SpatialDilatedConvolution_updateOutput(x, CT(), w4, None, CT(), CT(), 3, 3, 1, 1, 0, 0, 4, 4)


FULL_CASES = [
    # N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH, adjW, adjH
    (4, 16, 32, 14, 14, 4, 4, 2, 2, 1, 1, 1, 1, 0, 0),    # the usual 2x upsampling deconvolution
    (3, 32, 16, 12, 15, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1),    # output padding
    (2, 16, 16, 20, 20, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0),    # stride 1: forward through the flipped-weight kernel
    (2, 5, 7, 9, 11, 3, 2, 3, 2, 1, 0, 2, 2, 2, 1),       # rectangular, dilated, adj < stride
    (2, 8, 4, 10, 10, 5, 5, 1, 1, 0, 0, 2, 2, 0, 0),      # stride 1, dilated, no padding
    (2, 6, 10, 8, 8, 2, 2, 2, 2, 0, 0, 1, 1, 0, 0),       # k = stride: non-overlapping
]


def _full_run(T, case, bias=True, xt=None, scale=1.0, seed=90, dilated_entry=True, single=False):
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH = case
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cin, Cout, kH, kW)) * np.sqrt(2.0 / (Cin * kH * kW))).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32) if bias else None
    oargs = (kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH)
    if dilated_entry:
        fo, fg, fa = (THNN.SpatialFullDilatedConvolution_updateOutput, THNN.SpatialFullDilatedConvolution_updateGradInput,
                      THNN.SpatialFullDilatedConvolution_accGradParameters)
        args = oargs
    else:
        assert dlW == 1 and dlH == 1
        fo, fg, fa = (THNN.SpatialFullConvolution_updateOutput, THNN.SpatialFullConvolution_updateGradInput,
                      THNN.SpatialFullConvolution_accGradParameters)
        args = (kW, kH, dW, dH, pW, pH, aW, aH)
    xin = x[0] if single else x
    tx = xt(xin) if xt else CT.from_numpy(xin)
    tw, tb = CT.from_numpy(w), (CT.from_numpy(b) if bias else None)
    out, cols, ones = CT(), CT(), CT()
    fo(tx, out, tw, tb, cols, ones, *args)
    ry = O.fullconv_updateOutput(x, w, b, *oargs)
    y = out.numpy()
    assert y.shape == (ry[0].shape if single else ry.shape)
    close(y, ry[0] if single else ry)
    gy = rng.standard_normal(ry.shape).astype(np.float32)
    tgy = CT.from_numpy(gy[0] if single else gy)
    gi = CT()
    fg(tx, tgy, gi, tw, CT(), *args)
    rgi = O.fullconv_updateGradInput(x.shape, gy, w, *oargs)
    close(gi.numpy(), rgi[0] if single else rgi)
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    tgw, tgb = CT.from_numpy(gw0), (CT.from_numpy(gb0) if bias else None)
    fa(tx, tgy, tgw, tgb, cols, ones, *args, scale)
    rgw, rgb = O.fullconv_accGradParameters(x, gy, gw0.copy(), gb0.copy() if bias else None, *oargs, scale=scale)
    close(tgw.numpy(), rgw, WG_RTOL, WG_ATOL * max(1.0, abs(scale)) * 4)
    if bias:
        close(tgb.numpy(), rgb, WG_RTOL, WG_ATOL * max(1.0, abs(scale)) * 4)


@pytest.mark.parametrize("case", FULL_CASES)
def test_full_convolution(T, case):
    _full_run(T, case)


def test_full_convolution_phases_with_split_last_round(T):
    """The four phases of a 4x4 stride-2 transposed convolution run as one batched launch; with 392 tiles of
    128 x 128 and 48 k-tiles each on 256 CUs, the tiles past the first full round (the last images of the last
    two phases) are split along K and folded. First and last images against the oracle."""
    THNN, CT = T.THNN, T.CudaTensor
    N, Cin, Cout, H, k = 64, 192, 128, 14, 4
    rng = np.random.default_rng(92)
    x = rng.standard_normal((N, Cin, H, H)).astype(np.float32)
    w = (rng.standard_normal((Cin, Cout, k, k)) * np.sqrt(2.0 / (Cin * k * k))).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    out = CT()
    THNN.SpatialFullConvolution_updateOutput(CT.from_numpy(x), out, CT.from_numpy(w), CT.from_numpy(b), CT(), CT(),
                                             k, k, 2, 2, 1, 1, 0, 0)
    y = out.numpy()
    assert y.shape == (N, Cout, 2 * H, 2 * H)
    for n in (0, 1, 31, 32, 62, 63):
        close(y[n:n + 1], O.fullconv_updateOutput(x[n:n + 1], w, b, k, k, 2, 2, 1, 1, 1, 1, 0, 0))


def test_full_convolution_variants(T):
    rng = np.random.default_rng(91)
    _full_run(T, FULL_CASES[0], bias=False, scale=0.5, dilated_entry=False)
    _full_run(T, FULL_CASES[1], dilated_entry=False, xt=lambda a: T.CudaTensor.noncontiguous_from_numpy(a, rng), scale=2.0)
    _full_run(T, (1,) + FULL_CASES[2][1:], single=True, dilated_entry=False)
    cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", "1")
    try:
        _full_run(T, FULL_CASES[0])
        _full_run(T, FULL_CASES[2])
    finally:
        cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", None)


def test_full_convolution_errors(T):
    THNN, CT = T.THNN, T.CudaTensor
    x = CT.from_numpy(np.zeros((1, 4, 8, 8), np.float32))
    w = CT.from_numpy(np.zeros((4, 6, 3, 3), np.float32))
    with pytest.raises(T.THError, match="output padding must be smaller than either stride or dilation"):
        THNN.SpatialFullConvolution_updateOutput(x, CT(), w, None, CT(), CT(), 3, 3, 2, 2, 0, 0, 2, 0)
    with pytest.raises(T.THError, match="bias"):
        THNN.SpatialFullConvolution_updateOutput(x, CT(), w, CT.from_numpy(np.zeros(4, np.float32)), CT(), CT(),
                                                 3, 3, 1, 1, 0, 0, 0, 0)


TILE_CASES = [
    # both tile shapes of the forward and weight-gradient kernels (128 x 128, and 64 x 256 where that
    # wastes less of the tile): forward (rows = Cout), stride-1 gradInput (rows = Cin), gradWeight (Cout x K)
    (2, 40, 200, 20, 20, 3, 3, 1, 1, 1, 1, 1, 1),    # forward 128-row tiles, gradInput 64-row tiles
    (2, 192, 192, 12, 12, 3, 3, 1, 1, 1, 1, 1, 1),   # 192 rows = 3 x 64
    (2, 130, 70, 14, 18, 3, 3, 1, 1, 1, 1, 1, 1),    # gradInput: 130 rows, last 64-row tile holds 2
    (32, 16, 64, 48, 48, 3, 3, 1, 1, 1, 1, 1, 1),    # 64 rows, more tiles than CUs: full rounds + K-split tail
    (3, 3, 64, 40, 40, 7, 7, 2, 2, 3, 3, 1, 1),      # K = 147 padded to 160, stride 2
    (2, 24, 48, 18, 22, 3, 3, 1, 1, 1, 1, 1, 1),     # 64 x 256 weight-gradient tiles with L % 16 != 0
    # 64 x 64 weight-gradient tiles (the waves split the positions): narrow 1x1, first layers, L % 16 != 0,
    # Cout not a multiple of 4 (bias gradient in a pass of its own), 1x1 forward without a tap table
    (6, 32, 64, 28, 28, 1, 1, 1, 1, 0, 0, 1, 1),
    (4, 3, 32, 64, 64, 3, 3, 2, 2, 1, 1, 1, 1),
    (3, 5, 20, 18, 18, 3, 3, 1, 1, 1, 1, 1, 1),
    (2, 16, 27, 20, 24, 1, 1, 1, 1, 0, 0, 1, 1),
    (2, 48, 96, 12, 12, 1, 1, 1, 1, 0, 0, 1, 1),     # 1x1, K = 48: three k-tiles, computed tap offsets
]


@pytest.mark.parametrize("case", TILE_CASES)
def test_convolution_tile_shapes(T, case):
    _dil_run(T, case)


# gradInput (and the transposed convolution's forward pass) has two routes for geometries the flipped-weight
# forward kernel does not cover: one stride-1 GEMM per output phase (taken when Cin fills at least half of a
# 64-row tile) and gradient columns + col2im. Both are run on every geometry through the test switch.
PHASE_DIL_CASES = [c for c in DIL_CASES if c[7] != 1 or c[8] != 1 or c[9] > c[11] * (c[5] - 1)] + [
    (3, 64, 48, 23, 27, 3, 3, 2, 2, 1, 1, 1, 1),     # ResNet-style downsampling, odd extents
    (2, 40, 24, 17, 19, 5, 4, 3, 2, 2, 1, 1, 2),     # stride 3 x 2, rectangular, dilated rows
    (2, 33, 16, 16, 16, 1, 1, 2, 2, 0, 0, 1, 1),     # 1x1 stride 2: three of four phases have no tap at all
    (2, 32, 16, 15, 15, 2, 2, 4, 4, 0, 0, 1, 1),     # kernel smaller than the stride
    (2, 36, 20, 20, 21, 3, 3, 2, 2, 1, 1, 2, 2),     # stride 2 with dilation 2: only one phase per axis has taps
    (6, 128, 160, 14, 14, 3, 3, 2, 2, 1, 1, 1, 1),   # 128-row tiles, phases split along K
]


@pytest.mark.parametrize("route", ["phases", "columns"])
@pytest.mark.parametrize("case", PHASE_DIL_CASES)
def test_gradinput_routes(T, case, route):
    cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", route)
    try:
        _dil_run(T, case, seed=83)
    finally:
        cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", None)


@pytest.mark.parametrize("route", ["phases", "columns"])
@pytest.mark.parametrize("case", FULL_CASES + [(2, 24, 64, 9, 11, 4, 4, 2, 2, 1, 1, 1, 1, 0, 1)])
def test_full_convolution_routes(T, case, route):
    cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", route)
    try:
        _full_run(T, case, seed=92)
    finally:
        cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", None)


def _random_geometry(rng):
    while True:
        Cin = int(rng.choice([3, 17, 32, 48, 70, 130]))
        Cout = int(rng.choice([5, 33, 64, 100, 140]))
        kW, kH = (int(v) for v in rng.integers(1, 6, 2))
        dW, dH = (int(v) for v in rng.integers(1, 4, 2))
        pW, pH = (int(v) for v in rng.integers(0, 3, 2))
        dlW, dlH = (int(v) for v in rng.integers(1, 3, 2))
        H, W = (int(v) for v in rng.integers(6, 25, 2))
        if H + 2 * pH >= dlH * (kH - 1) + 1 and W + 2 * pW >= dlW * (kW - 1) + 1:
            return (int(rng.integers(1, 4)), Cin, Cout, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH)


@pytest.mark.parametrize("seed", range(24))
def test_convolution_random_geometries(T, seed):
    """Seeded draws over kernel size, stride, padding, dilation and channel counts on either side of the
    tile-shape and gradInput-route thresholds; the gradInput route alternates between the default choice,
    the phase route and the column route."""
    rng = np.random.default_rng(1000 + seed)
    case = _random_geometry(rng)
    route = [None, "phases", "columns"][seed % 3]
    if route:
        cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", route)
    try:
        _dil_run(T, case, seed=2000 + seed, scale=float(rng.choice([1.0, 0.5])))
    finally:
        cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", None)

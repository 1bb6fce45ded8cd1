"""GPU parity: every THNN_Cuda* entry point, called through the C ABI, against the
CPU oracle on the same seeded inputs. Mirrors what test.lua does for the five
module families (random shapes from the reference's ranges, contiguous and
non-contiguous inputs, with/without bias, ceil_mode on/off, include/exclude pad,
BN train/eval and fused/split backward, accumulation into non-zero gradients).

Tolerances (stated by the task): 1e-5 relative / 1e-4 absolute for fp32 outputs
and gradients; 1e-3 relative for weight gradients and BN batch statistics;
max-pool argmax indices bit-exact.
"""
import os

import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402

OUT_RTOL, OUT_ATOL = 1e-5, 1e-4
WG_RTOL, WG_ATOL = 1e-3, 1e-4


@pytest.fixture(scope="module")
def T():
    import cunn_amd
    return cunn_amd


def close(a, b, rtol=OUT_RTOL, atol=OUT_ATOL):
    np.testing.assert_allclose(a, b, rtol=rtol, atol=atol)


class force_direct:
    """Routes a call to the shape-agnostic kernels ("1") or, for the depthwise
    convolution, to the generic LDS-tiled kernels ("2") instead of the fastest path."""

    def __init__(self, var, mode="1"):
        self.var, self.mode = var, mode

    def __enter__(self):
        cunn_amd.set_switch(self.var, self.mode)

    def __exit__(self, *a):
        cunn_amd.set_switch(self.var, None)


# ------------------------------------------------------------------ depthwise --
DW_CASES = [
    # N, C, M, H, W, kW, kH, dW, dH, padW, padH
    (3, 3, 4, 28, 28, 3, 3, 1, 1, 1, 1),     # the reference's own test shape (test.lua:6639-6645)
    (4, 8, 1, 56, 56, 3, 3, 2, 2, 1, 1),     # headline geometry, small batch
    (2, 5, 1, 112, 112, 3, 3, 1, 1, 1, 1),   # first MobileNet depthwise layer geometry
    (2, 4, 2, 30, 34, 5, 5, 1, 1, 2, 2),
    (2, 4, 1, 31, 33, 5, 5, 2, 2, 2, 2),     # odd width: scalar loaders
    (1, 3, 2, 17, 19, 3, 2, 2, 1, 0, 1),     # rectangular kernel/stride: runtime geometry
    (2, 2, 3, 9, 40, 4, 4, 3, 3, 1, 1),
    (1, 6, 1, 7, 7, 3, 3, 1, 1, 1, 1),       # tiny planes
    (2, 2, 1, 150, 260, 3, 3, 1, 1, 1, 1),   # several row bands per plane
    (1, 2, 1, 12, 12, 7, 7, 2, 2, 3, 3),
    (2, 3, 2, 24, 32, 5, 5, 1, 1, 2, 2),     # 5x5 strip kernels
    (2, 3, 1, 40, 48, 5, 5, 2, 2, 2, 2),
    (2, 3, 2, 57, 56, 3, 3, 2, 2, 1, 1),     # odd height under stride 2
    (1, 2, 1, 8, 8, 3, 3, 2, 2, 1, 1),
]


def _dw_inputs(case, seed, bias=True):
    N, C, M, H, W, kW, kH, dW, dH, pW, pH = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    bound = np.sqrt(6.0 / (kH * kW))
    w = rng.uniform(-bound, bound, (M, C, kH, kW)).astype(np.float32)
    b = rng.uniform(-0.3, 0.3, (M, C)).astype(np.float32) if bias else None
    return rng, x, w, b


def _dw_run(T, case, x, w, b, gy_seed=7, xt=None, scale=1.0, gw0=None, gb0=None):
    N, C, M, H, W, kW, kH, dW, dH, pW, pH = case
    THNN, CT = T.THNN, T.CudaTensor
    tx = xt if xt is not None else CT.from_numpy(x)
    tw = CT.from_numpy(w)
    tb = CT.from_numpy(b) if b is not None else None
    out, cols, ones = CT(), CT(), CT()
    THNN.SpatialDepthWiseConvolution_updateOutput(tx, out, tw, tb, cols, ones, kW, kH, dW, dH, pW, pH)
    y = out.numpy()
    ry = O.dwconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH)
    assert y.shape == ry.shape
    close(y, ry)
    gy = np.random.default_rng(gy_seed).standard_normal(y.shape).astype(np.float32)
    tgy, gi = CT.from_numpy(gy), CT()
    THNN.SpatialDepthWiseConvolution_updateGradInput(tx, tgy, gi, tw, cols, ones, kW, kH, dW, dH, pW, pH)
    close(gi.numpy(), O.dwconv_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH))
    gw0 = np.zeros_like(w) if gw0 is None else gw0
    gb0 = np.zeros((M, C), np.float32) if gb0 is None else gb0
    tgw = CT.from_numpy(gw0)
    tgb = CT.from_numpy(gb0) if b is not None else None
    THNN.SpatialDepthWiseConvolution_accGradParameters(tx, tgy, tgw, tgb, cols, ones, kW, kH, dW, dH, pW, pH, scale)
    rgw, rgb = O.dwconv_accGradParameters(x, gy, gw0.copy(), gb0.copy() if b is not None else None,
                                          kW, kH, dW, dH, pW, pH, scale)
    close(tgw.numpy(), rgw, WG_RTOL, WG_ATOL)
    if b is not None:
        close(tgb.numpy(), rgb, WG_RTOL, WG_ATOL)
    return y


@pytest.mark.parametrize("case", DW_CASES)
def test_dwconv_tiled(T, case):
    _, x, w, b = _dw_inputs(case, 1)
    _dw_run(T, case, x, w, b)


@pytest.mark.parametrize("case", DW_CASES[:7] + DW_CASES[10:12])
@pytest.mark.parametrize("mode", ["1", "2"])
def test_dwconv_fallback_kernels(T, case, mode):
    _, x, w, b = _dw_inputs(case, 2)
    with force_direct("THCUNN_DW_FORCE_DIRECT", mode):
        _dw_run(T, case, x, w, b)


DW_SMALL_CASES = [
    # planes of at most 1024 elements with depth multiplier 1: several planes per workgroup
    (4, 40, 1, 14, 14, 3, 3, 1, 1, 1, 1),    # MobileNet 14x14 stage: 16 planes per workgroup, 7 outputs per item
    (4, 40, 1, 14, 14, 3, 3, 2, 2, 1, 1),    # 14 -> 7
    (3, 70, 1, 7, 7, 3, 3, 1, 1, 1, 1),      # 7x7: 64 planes per workgroup, last workgroup partly filled
    (2, 24, 1, 28, 28, 3, 3, 2, 2, 1, 1),    # 28 -> 14: width fits the strip kernels, output width does not
    (3, 10, 1, 28, 28, 5, 5, 2, 2, 2, 2),    # 5x5
    (2, 12, 1, 14, 14, 5, 5, 1, 1, 2, 2),
    (3, 5, 1, 13, 11, 3, 3, 1, 1, 1, 1),     # odd extents: 4 outputs per item with a masked tail
    (2, 6, 1, 15, 18, 3, 3, 2, 2, 1, 1),     # odd height under stride 2: the last input row is never read
    (1, 3, 1, 5, 5, 3, 3, 2, 2, 1, 1),       # three planes in all: one workgroup, mostly idle
    (5, 16, 1, 31, 31, 3, 3, 2, 2, 1, 1),    # 961 elements: 4 planes per workgroup
    (2, 8, 1, 9, 9, 5, 5, 2, 2, 2, 2),
    (1, 4, 1, 2, 2, 3, 3, 1, 1, 1, 1),       # plane smaller than the kernel
]


@pytest.mark.parametrize("case", DW_SMALL_CASES)
def test_dwconv_small_planes(T, case):
    rng, x, w, b = _dw_inputs(case, 11)
    _dw_run(T, case, x, w, b, scale=0.5, gw0=rng.standard_normal(w.shape).astype(np.float32),
            gb0=rng.standard_normal((case[2], case[1])).astype(np.float32))


@pytest.mark.parametrize("case", [DW_CASES[0][:2] + (1,) + DW_CASES[0][3:], (2, 6, 1, 16, 16, 3, 3, 1, 1, 1, 1),
                                  (2, 6, 1, 32, 32, 3, 3, 2, 2, 1, 1), (2, 6, 1, 24, 32, 5, 5, 1, 1, 2, 2)])
@pytest.mark.parametrize("switch", ["0", "1"])
def test_dwconv_small_planes_switch(T, case, switch):
    """Shapes both kernel families take: "0" hands them to the strip kernels, "1" leaves the default (small-plane kernels)."""
    _, x, w, b = _dw_inputs(case, 12)
    with force_direct("THCUNN_DW_SMALL", switch):
        _dw_run(T, case, x, w, b)


def test_dwconv_small_planes_special_values(T):
    """A work item whose last outputs are masked off (width 6, 4 outputs per item) reads past the end of its row;
    what it finds there - here an infinity in column 0 of the next row - must not reach any sum."""
    case = (2, 8, 1, 6, 6, 3, 3, 1, 1, 1, 1)
    _, x, w, b = _dw_inputs(case, 13)
    x[0, 3, 2, 0] = np.inf
    THNN, CT = T.THNN, T.CudaTensor
    out = CT()
    THNN.SpatialDepthWiseConvolution_updateOutput(CT.from_numpy(x), out, CT.from_numpy(w), CT.from_numpy(b), CT(), CT(),
                                                  3, 3, 1, 1, 1, 1)
    y = out.numpy()
    with np.errstate(invalid="ignore"):
        ry = O.dwconv_updateOutput(x, w, b, 3, 3, 1, 1, 1, 1)
    assert np.array_equal(np.isfinite(y), np.isfinite(ry))
    close(y[np.isfinite(ry)], ry[np.isfinite(ry)])
    gy = np.random.default_rng(14).standard_normal(y.shape).astype(np.float32)
    gw, gb = CT.from_numpy(np.zeros_like(w)), CT.from_numpy(np.zeros_like(b))
    THNN.SpatialDepthWiseConvolution_accGradParameters(CT.from_numpy(x), CT.from_numpy(gy), gw, gb, CT(), CT(),
                                                       3, 3, 1, 1, 1, 1, 1.0)
    with np.errstate(invalid="ignore"):
        rgw, rgb = O.dwconv_accGradParameters(x, gy, np.zeros_like(w), np.zeros_like(b), 3, 3, 1, 1, 1, 1, 1.0)
    g = gw.numpy()
    fin = np.isfinite(rgw)
    assert fin[0, 3, :, 2].all() and not fin[0, 3, :, 0].all()   # column 0 of the input never meets tap column 2
    assert np.array_equal(np.isfinite(g), fin)
    close(g[fin], rgw[fin], WG_RTOL, WG_ATOL)
    close(gb.numpy(), rgb, WG_RTOL, WG_ATOL)


def test_dwconv_accgrad_deterministic(T):
    """accGradParameters folds per-workgroup partials in a fixed order (no atomics): repeated
    calls on the same inputs are bit-identical."""
    THNN, CT = T.THNN, T.CudaTensor
    case = (6, 40, 1, 56, 56, 3, 3, 2, 2, 1, 1)
    N, C, M, H, W, kW, kH, dW, dH, pW, pH = case
    rng, x, w, b = _dw_inputs(case, 9)
    oH = (H + 2 * pH - kH) // dH + 1
    gy = rng.standard_normal((N, C, oH, oH)).astype(np.float32)
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    gb0 = rng.standard_normal(b.shape).astype(np.float32)
    rgw, rgb = O.dwconv_accGradParameters(x, gy, gw0.copy(), gb0.copy(), kW, kH, dW, dH, pW, pH, 0.5)

    def run():
        tgw, tgb = CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.SpatialDepthWiseConvolution_accGradParameters(CT.from_numpy(x), CT.from_numpy(gy), tgw, tgb, CT(), CT(),
                                                           kW, kH, dW, dH, pW, pH, 0.5)
        return tgw.numpy(), tgb.numpy()

    results = [run() for _ in range(3)]
    for gw, gb in results:
        close(gw, rgw, WG_RTOL, WG_ATOL)
        close(gb, rgb, WG_RTOL, WG_ATOL)
        assert np.array_equal(gw, results[0][0]) and np.array_equal(gb, results[0][1])


def test_dwconv_no_bias_scale_and_accumulate(T):
    case = (3, 6, 2, 20, 24, 3, 3, 2, 2, 1, 1)
    rng, x, w, _ = _dw_inputs(case, 3, bias=False)
    _dw_run(T, case, x, w, None, scale=0.25, gw0=rng.standard_normal(w.shape).astype(np.float32))
    rng, x, w, b = _dw_inputs(case, 4)
    _dw_run(T, case, x, w, b, scale=-1.5, gw0=rng.standard_normal(w.shape).astype(np.float32),
            gb0=rng.standard_normal(b.shape).astype(np.float32))


def test_dwconv_noncontiguous_input(T):
    case = (3, 4, 2, 18, 20, 3, 3, 1, 1, 1, 1)
    rng, x, w, b = _dw_inputs(case, 5)
    xt = T.CudaTensor.noncontiguous_from_numpy(x, rng)
    assert not xt.is_contiguous()
    _dw_run(T, case, x, w, b, xt=xt)


def test_dwconv_single_image_and_2d_weight(T):
    """3-D input gives a 3-D output; a 2-D (M, C*kH*kW) weight is reshaped to 4-D in
    place on the caller's tensor (generic/SpatialDepthWiseConvolution.cu:76-80)."""
    THNN, CT = T.THNN, T.CudaTensor
    C, M, H, W, k = 5, 3, 14, 16, 3
    rng = np.random.default_rng(6)
    x = rng.standard_normal((C, H, W)).astype(np.float32)
    w = rng.standard_normal((M, C, k, k)).astype(np.float32)
    b = rng.standard_normal((M, C)).astype(np.float32)
    tw = CT.from_numpy(w.reshape(M, C * k * k))
    out = CT()
    THNN.SpatialDepthWiseConvolution_updateOutput(CT.from_numpy(x), out, tw, CT.from_numpy(b), CT(), CT(), k, k, 1, 1, 1, 1)
    assert tw.size() == (M, C, k, k)
    y = out.numpy()
    assert y.shape == (C * M, H, W)
    close(y, O.dwconv_updateOutput(x[None], w, b, k, k, 1, 1, 1, 1)[0])
    gy = rng.standard_normal(y.shape).astype(np.float32)
    gi = CT()
    THNN.SpatialDepthWiseConvolution_updateGradInput(CT.from_numpy(x), CT.from_numpy(gy), gi, tw, CT(), CT(), k, k, 1, 1, 1, 1)
    assert gi.size() == (C, H, W)
    close(gi.numpy(), O.dwconv_updateGradInput((1, C, H, W), gy[None], w, k, k, 1, 1, 1, 1)[0])


def test_dwconv_transposed_gradweight_view(T):
    """gradWeight is written through its strides: a (M, C, kH, kW) view of (C, M, kH, kW)
    memory - what the reference leaves behind after a call (:619-629) - accumulates correctly."""
    THNN, CT = T.THNN, T.CudaTensor
    case = (2, 4, 3, 12, 12, 3, 3, 1, 1, 1, 1)
    N, C, M, H, W, k = 2, 4, 3, 12, 12, 3
    rng, x, w, b = _dw_inputs(case, 8)
    gy = rng.standard_normal((N, C * M, H, W)).astype(np.float32)
    gw0 = rng.standard_normal((M, C, k, k)).astype(np.float32)
    base = CT.from_numpy(np.ascontiguousarray(gw0.transpose(1, 0, 2, 3)))       # memory in (C, M, k, k) order
    view = base.view(0, (M, C, k, k), (k * k, M * k * k, k, 1))
    THNN.SpatialDepthWiseConvolution_accGradParameters(CT.from_numpy(x), CT.from_numpy(gy), view, None, CT(), CT(),
                                                       k, k, 1, 1, 1, 1, 1.0)
    rgw, _ = O.dwconv_accGradParameters(x, gy, gw0.copy(), None, k, k, 1, 1, 1, 1, 1.0)
    close(base.numpy().transpose(1, 0, 2, 3), rgw, WG_RTOL, WG_ATOL)


def test_dwconv_small_planes_variants(T):
    """The several-planes-per-workgroup kernels behind the other ways of calling the module: no bias, a
    non-contiguous input, a 3-D input with a 2-D weight, gradWeight and gradBias through transposed views."""
    THNN, CT = T.THNN, T.CudaTensor
    case = (3, 20, 1, 14, 14, 3, 3, 2, 2, 1, 1)
    rng, x, w, _ = _dw_inputs(case, 15, bias=False)
    _dw_run(T, case, x, w, None, scale=2.0, gw0=rng.standard_normal(w.shape).astype(np.float32))
    rng, x, w, b = _dw_inputs(case, 16)
    _dw_run(T, case, x, w, b, xt=CT.noncontiguous_from_numpy(x, rng))
    # 3-D input, 2-D weight
    C, H, W, k = 20, 7, 7, 3
    x3 = rng.standard_normal((C, H, W)).astype(np.float32)
    w4 = rng.standard_normal((1, C, k, k)).astype(np.float32)
    b2 = rng.standard_normal((1, C)).astype(np.float32)
    tw, out = CT.from_numpy(w4.reshape(1, C * k * k)), CT()
    THNN.SpatialDepthWiseConvolution_updateOutput(CT.from_numpy(x3), out, tw, CT.from_numpy(b2), CT(), CT(), k, k, 1, 1, 1, 1)
    assert out.size() == (C, H, W)
    close(out.numpy(), O.dwconv_updateOutput(x3[None], w4, b2, k, k, 1, 1, 1, 1)[0])
    gy3 = rng.standard_normal((C, H, W)).astype(np.float32)
    gi = CT()
    THNN.SpatialDepthWiseConvolution_updateGradInput(CT.from_numpy(x3), CT.from_numpy(gy3), gi, tw, CT(), CT(), k, k, 1, 1, 1, 1)
    assert gi.size() == (C, H, W)
    close(gi.numpy(), O.dwconv_updateGradInput((1, C, H, W), gy3[None], w4, k, k, 1, 1, 1, 1)[0])
    # gradWeight as a (1, C, k, k) view of memory in (C, k, k) order with a gap between channels; gradBias likewise
    gw0 = rng.standard_normal((1, C, k, k)).astype(np.float32)
    basew = CT.from_numpy(np.zeros((C, 2 * k * k), np.float32))
    hw = basew.numpy(); hw[:, :k * k] = gw0[0].reshape(C, k * k)
    basew = CT.from_numpy(hw)
    vieww = basew.view(0, (1, C, k, k), (0, 2 * k * k, k, 1))
    gb0 = rng.standard_normal((1, C)).astype(np.float32)
    THNN.SpatialDepthWiseConvolution_accGradParameters(CT.from_numpy(x3), CT.from_numpy(gy3), vieww, CT.from_numpy(gb0.copy()),
                                                       CT(), CT(), k, k, 1, 1, 1, 1, 0.5)
    rgw, _ = O.dwconv_accGradParameters(x3[None], gy3[None], gw0.copy(), gb0.copy(), k, k, 1, 1, 1, 1, 0.5)
    got = basew.numpy()
    close(got[:, :k * k].reshape(1, C, k, k), rgw, WG_RTOL, WG_ATOL)
    assert np.all(got[:, k * k:] == 0)


def test_dwconv_shape_errors(T):
    THNN, CT = T.THNN, T.CudaTensor
    x = CT.from_numpy(np.zeros((2, 3, 8, 8), np.float32))
    w = CT.from_numpy(np.zeros((1, 4, 3, 3), np.float32))   # 4 planes vs 3 in the input
    with pytest.raises(T.THError, match="Need input of dimension 4"):
        THNN.SpatialDepthWiseConvolution_updateOutput(x, CT(), w, None, CT(), CT(), 3, 3, 1, 1, 1, 1)
    w = CT.from_numpy(np.zeros((1, 3, 3, 3), np.float32))
    with pytest.raises(T.THError, match="stride should be greater than zero"):
        THNN.SpatialDepthWiseConvolution_updateOutput(x, CT(), w, None, CT(), CT(), 3, 3, 0, 1, 1, 1)
    big = CT.from_numpy(np.zeros((1, 3, 11, 11), np.float32))
    with pytest.raises(T.THError, match="Output size is too small"):
        THNN.SpatialDepthWiseConvolution_updateOutput(x, CT(), big, None, CT(), CT(), 11, 11, 1, 1, 0, 0)


# -------------------------------------------------------------------- pooling --
POOL_CASES = [
    # N, C, H, W, kW, kH, dW, dH, padW, padH, ceil
    (2, 3, 112, 112, 3, 3, 2, 2, 1, 1, False),   # headline max-pool geometry
    (2, 3, 112, 112, 2, 2, 2, 2, 0, 0, False),   # headline avg-pool geometry
    (3, 4, 33, 37, 3, 3, 2, 2, 1, 1, True),
    (2, 2, 40, 41, 2, 3, 2, 1, 1, 0, True),
    (2, 5, 64, 64, 4, 4, 4, 4, 2, 2, True),
    (1, 2, 65, 47, 4, 2, 3, 2, 0, 1, False),
    (4, 7, 32, 32, 3, 3, 1, 1, 1, 1, False),
    (1, 1, 5, 5, 2, 2, 1, 1, 1, 1, False),
    (1, 2, 300, 260, 3, 3, 2, 2, 1, 1, False),   # several row bands per plane
    (2, 3, 48, 48, 3, 3, 2, 2, 0, 0, True),      # unpadded 3x3 s2, ceil mode: last window overhangs
    (1, 2, 300, 264, 3, 3, 2, 2, 1, 1, False),   # strip kernels, several bands
    (2, 2, 31, 40, 3, 3, 1, 1, 1, 1, False),     # 3x3 s1 strip with odd height
    (3, 2, 27, 48, 3, 3, 3, 3, 0, 0, False),     # window = stride 3, exact tiling (flat average kernels)
    (2, 3, 40, 64, 4, 4, 4, 4, 0, 0, True),      # window = stride 4, exact tiling, ceil mode without effect
    (2, 2, 22, 24, 2, 2, 2, 2, 0, 0, False),     # window = stride 2, oW = 12
]


def _tied_input(shape, seed, q=64):
    return (np.round(np.random.default_rng(seed).uniform(-1, 1, shape) * q) / q).astype(np.float32)


def _maxpool_run(T, case, x, dil=(1, 1), xt=None):
    N, C, H, W, kW, kH, dW, dH, pW, pH, ceil = case
    THNN, CT, LT = T.THNN, T.CudaTensor, T.CudaLongTensor
    tx = xt if xt is not None else CT.from_numpy(x)
    out, idx = CT(), LT()
    if dil == (1, 1):
        THNN.SpatialMaxPooling_updateOutput(tx, out, idx, kW, kH, dW, dH, pW, pH, ceil)
    else:
        THNN.SpatialDilatedMaxPooling_updateOutput(tx, out, idx, kW, kH, dW, dH, pW, pH, dil[0], dil[1], ceil)
    ry, ridx = O.maxpool_updateOutput(x, kW, kH, dW, dH, pW, pH, ceil, dil[0], dil[1])
    y, i = out.numpy(), idx.numpy()
    assert y.shape == ry.shape and i.dtype == np.int64
    assert np.array_equal(y, ry)
    assert np.array_equal(i, ridx)                       # bit-exact argmax, 1-based
    gy = np.random.default_rng(11).standard_normal(y.shape).astype(np.float32)
    gi = CT()
    if dil == (1, 1):
        THNN.SpatialMaxPooling_updateGradInput(tx, CT.from_numpy(gy), gi, idx, kW, kH, dW, dH, pW, pH, ceil)
    else:
        THNN.SpatialDilatedMaxPooling_updateGradInput(tx, CT.from_numpy(gy), gi, idx, kW, kH, dW, dH, pW, pH,
                                                      dil[0], dil[1], ceil)
    rgi = O.maxpool_updateGradInput(x.shape, gy, ridx, kW, kH, dW, dH, pW, pH, ceil, dil[0], dil[1])
    close(gi.numpy(), rgi)


@pytest.mark.parametrize("case", POOL_CASES)
def test_maxpool_ties_bit_exact(T, case):
    _maxpool_run(T, case, _tied_input(case[:4], 20))


@pytest.mark.parametrize("case", POOL_CASES[:6] + POOL_CASES[9:10])
@pytest.mark.parametrize("mode", ["1", "2"])
def test_maxpool_fallback_kernels(T, case, mode):
    with force_direct("THCUNN_POOL_FORCE_DIRECT", mode):
        _maxpool_run(T, case, _tied_input(case[:4], 21, q=8))


POOL_SMALL_CASES = [
    # planes of at most 1024 elements outside the strip kernels' geometries: several planes per workgroup
    (4, 40, 14, 14, 2, 2, 2, 2, 0, 0, False),    # VGG-style 14 -> 7
    (3, 33, 28, 28, 2, 2, 2, 2, 0, 0, False),    # 28 -> 14: plane count not a multiple of the group
    (2, 20, 13, 13, 3, 3, 2, 2, 0, 0, False),    # overlapping 3x3 stride 2, odd plane
    (2, 12, 27, 27, 3, 3, 2, 2, 0, 0, True),     # ceil mode
    (2, 9, 7, 7, 3, 3, 1, 1, 1, 1, False),       # padded, stride 1
    (3, 5, 15, 9, 2, 3, 1, 2, 1, 0, True),       # rectangular everything
    (1, 3, 6, 6, 3, 3, 2, 2, 1, 1, False),       # three planes in all
    (2, 70, 5, 5, 2, 2, 2, 2, 0, 0, True),       # ceil mode with a clipped last window
    (300, 9, 3, 3, 2, 2, 1, 1, 0, 0, False),     # many tiny planes
]


@pytest.mark.parametrize("case", POOL_SMALL_CASES)
def test_maxpool_small_planes(T, case):
    _maxpool_run(T, case, _tied_input(case[:4], 25, q=8))
    if case[4] > 1 and case[5] > 1 and case[2] >= 9 and case[3] >= 9:
        _maxpool_run(T, case, _tied_input(case[:4], 26, q=8), dil=(2, 2))


@pytest.mark.parametrize("case", POOL_SMALL_CASES)
@pytest.mark.parametrize("include_pad", [True, False])
def test_avgpool_small_planes(T, case, include_pad):
    _avgpool_run(T, case, include_pad, seed=34)


def test_maxpool_dilated_and_noncontiguous(T):
    case = (2, 3, 30, 34, 3, 2, 2, 1, 1, 1, False)
    x = _tied_input(case[:4], 22, q=16)
    _maxpool_run(T, case, x, dil=(2, 3))
    rng = np.random.default_rng(23)
    _maxpool_run(T, case, x, xt=T.CudaTensor.noncontiguous_from_numpy(x, rng))


def test_maxpool_single_image_and_nan(T):
    THNN, CT, LT = T.THNN, T.CudaTensor, T.CudaLongTensor
    x = _tied_input((3, 10, 12), 24)
    out, idx = CT(), LT()
    THNN.SpatialMaxPooling_updateOutput(CT.from_numpy(x), out, idx, 2, 2, 2, 2, 0, 0, False)
    assert out.size() == (3, 5, 6) and idx.size() == (1, 3, 5, 6)   # indices stay 4-D (:140-141)
    ry, ridx = O.maxpool_updateOutput(x[None], 2, 2, 2, 2, 0, 0, False)
    assert np.array_equal(out.numpy(), ry[0]) and np.array_equal(idx.numpy(), ridx)
    xn = np.full((1, 1, 2, 2), np.nan, np.float32)
    THNN.SpatialMaxPooling_updateOutput(CT.from_numpy(xn), out, idx, 2, 2, 2, 2, 0, 0, False)
    assert out.numpy()[0, 0, 0, 0] == -np.finfo(np.float32).max and idx.numpy()[0, 0, 0, 0] == 0


def test_pool_errors(T):
    THNN, CT, LT = T.THNN, T.CudaTensor, T.CudaLongTensor
    x = CT.from_numpy(np.zeros((1, 1, 8, 8), np.float32))
    with pytest.raises(T.THError, match="pad should be smaller than half of kernel size"):
        THNN.SpatialMaxPooling_updateOutput(x, CT(), LT(), 2, 2, 2, 2, 2, 2, False)
    with pytest.raises(T.THError, match="pad should be smaller than half of kernel size"):
        THNN.SpatialAveragePooling_updateOutput(x, CT(), 2, 2, 2, 2, 2, 2, False, True)


def _avgpool_run(T, case, include_pad, xt=None, seed=30):
    N, C, H, W, kW, kH, dW, dH, pW, pH, ceil = case
    THNN, CT = T.THNN, T.CudaTensor
    x = np.random.default_rng(seed).standard_normal((N, C, H, W)).astype(np.float32)
    tx = xt(x) if xt else CT.from_numpy(x)
    out = CT()
    THNN.SpatialAveragePooling_updateOutput(tx, out, kW, kH, dW, dH, pW, pH, ceil, include_pad)
    ry = O.avgpool_updateOutput(x, kW, kH, dW, dH, pW, pH, ceil, include_pad)
    close(out.numpy(), ry)
    gy = np.random.default_rng(seed + 1).standard_normal(ry.shape).astype(np.float32)
    gi = CT()
    THNN.SpatialAveragePooling_updateGradInput(tx, CT.from_numpy(gy), gi, kW, kH, dW, dH, pW, pH, ceil, include_pad)
    close(gi.numpy(), O.avgpool_updateGradInput(x.shape, gy, kW, kH, dW, dH, pW, pH, ceil, include_pad))


@pytest.mark.parametrize("case", POOL_CASES)
@pytest.mark.parametrize("include_pad", [True, False])
def test_avgpool(T, case, include_pad):
    _avgpool_run(T, case, include_pad)


@pytest.mark.parametrize("case", POOL_CASES[:6])
def test_avgpool_direct_and_noncontiguous(T, case):
    for mode in ("1", "2"):
        with force_direct("THCUNN_POOL_FORCE_DIRECT", mode):
            _avgpool_run(T, case, True)
            _avgpool_run(T, case, False)
    rng = np.random.default_rng(31)
    _avgpool_run(T, case, True, xt=lambda a: T.CudaTensor.noncontiguous_from_numpy(a, rng))


@pytest.mark.parametrize("case", [
    (5, 37, 7, 7, 7, 7, 1, 1, 0, 0, False),      # global pooling of a 7x7 plane; plane count not a multiple of 4
    (2, 3, 13, 9, 9, 13, 1, 1, 0, 0, True),      # rectangular plane of more than 64 elements, ceil mode
    (1, 1, 1, 1, 1, 1, 1, 1, 0, 0, False),       # a single element
    (3, 6, 8, 8, 8, 8, 8, 8, 0, 0, False),       # stride = window
])
@pytest.mark.parametrize("include_pad", [True, False])
def test_avgpool_global(T, case, include_pad):
    _avgpool_run(T, case, include_pad, seed=33)
    with force_direct("THCUNN_POOL_FORCE_DIRECT", "2"):
        _avgpool_run(T, case, include_pad, seed=33)


def test_avgpool_reference_known_answer(T):
    """test.lua:2597-2616 through the C ABI: 1x1x1x1 input 3, k2 s1 p1 -> 3 and 3/4."""
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(32)
    x = np.full((1, 1, 1, 1), 3.0, np.float32)
    tx = CT.noncontiguous_from_numpy(x, rng)
    a, b = CT(), CT()
    THNN.SpatialAveragePooling_updateOutput(tx, a, 2, 2, 1, 1, 1, 1, False, False)
    THNN.SpatialAveragePooling_updateOutput(tx, b, 2, 2, 1, 1, 1, 1, False, True)
    assert a.numpy()[0, 0, 0, 0] == 3.0 and b.numpy()[0, 0, 0, 0] == 0.75


# ------------------------------------------------------------------------- BN --
BN_SHAPES = [(8, 16, 28, 28), (4, 3, 7, 5), (32, 64), (2, 5, 33), (3, 2, 4, 5, 6), (2, 2, 150, 120), (1, 3, 9000),
             # channel-resident kernels (C >= 96, a channel fits one workgroup's registers)
             (64, 100, 28, 28), (40, 96, 20, 20), (33, 97, 12, 12), (4, 128, 14, 14), (57, 96, 24, 28),
             # small channels with planes that are not a multiple of 4 elements (scalar resident kernels)
             (16, 130, 7, 7), (64, 96, 7, 7), (5, 100, 3, 3), (160, 97, 7, 7), (3, 128, 1, 1), (2, 96, 13, 11)]


def _bn_run(T, shape, affine, seed=40):
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(seed)
    Cc = shape[1]
    x = (rng.standard_normal(shape) * 2 + 0.5 + np.arange(Cc).reshape((1, Cc) + (1,) * (len(shape) - 2))).astype(np.float32)
    g = rng.random(Cc).astype(np.float32) if affine else None
    b = rng.standard_normal(Cc).astype(np.float32) if affine else None
    rm0 = rng.standard_normal(Cc).astype(np.float32)
    rv0 = (rng.random(Cc) + 0.5).astype(np.float32)
    eps, mom = 1e-5, 0.1
    tx = CT.from_numpy(x)
    tg = CT.from_numpy(g) if affine else None
    tb = CT.from_numpy(b) if affine else None
    trm, trv, tsm, tss, out = CT.from_numpy(rm0), CT.from_numpy(rv0), CT.with_size(Cc), CT.with_size(Cc), CT()
    THNN.BatchNormalization_updateOutput(tx, out, tg, tb, trm, trv, tsm, tss, True, mom, eps)
    rm, rv = rm0.copy(), rv0.copy()
    ry, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, mom, eps)
    assert out.size() == tuple(shape)
    close(out.numpy(), ry)
    close(tsm.numpy(), sm, WG_RTOL, 1e-5)
    close(tss.numpy(), ss, WG_RTOL, 1e-6)
    close(trm.numpy(), rm, WG_RTOL, 1e-5)
    close(trv.numpy(), rv, WG_RTOL, 1e-5)
    # evaluation mode
    oute = CT()
    THNN.BatchNormalization_updateOutput(tx, oute, tg, tb, trm, trv, tsm, tss, False, mom, eps)
    rye, _, _ = O.bn_updateOutput(x, g, b, rm.copy(), rv.copy(), False, mom, eps)
    close(oute.numpy(), rye)
    # backward: fused call, then the split order (updateGradInput, accGradParameters) (test.lua:989-1003)
    gy = rng.standard_normal(shape).astype(np.float32)
    tgy = CT.from_numpy(gy)
    gw0 = rng.standard_normal(Cc).astype(np.float32)
    gb0 = rng.standard_normal(Cc).astype(np.float32)
    for train in (True, False):
        gi = CT.with_size(*shape)
        tgw, tgb = CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.BatchNormalization_backward(tx, tgy, gi, tgw, tgb, tg, trm, trv, tsm, tss, train, 0.5, eps)
        rgi, rgw, rgb = O.bn_backward(x, gy, g, rm, rv, sm, ss, train, 0.5, eps, gw0.copy(), gb0.copy())
        close(gi.numpy(), rgi)
        close(tgw.numpy(), rgw, WG_RTOL, 1e-3)
        close(tgb.numpy(), rgb, WG_RTOL, 1e-3)
        gi2 = CT.with_size(*shape)
        THNN.BatchNormalization_backward(tx, tgy, gi2, None, None, tg, trm, trv, tsm, tss, train, 0.5, eps)
        tgw2, tgb2 = CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.BatchNormalization_backward(tx, tgy, None, tgw2, tgb2, tg, trm, trv, tsm, tss, train, 0.5, eps)
        assert np.array_equal(gi.numpy(), gi2.numpy())
        assert np.array_equal(tgw.numpy(), tgw2.numpy()) and np.array_equal(tgb.numpy(), tgb2.numpy())


@pytest.mark.parametrize("shape", BN_SHAPES)
@pytest.mark.parametrize("affine", [True, False])
def test_batchnorm(T, shape, affine):
    _bn_run(T, shape, affine)


def test_batchnorm_chunked_path_on_resident_shape(T):
    cunn_amd.set_switch("THCUNN_BN_FORCE_CHUNKED", "1")
    try:
        _bn_run(T, (40, 96, 20, 20), True)
    finally:
        cunn_amd.set_switch("THCUNN_BN_FORCE_CHUNKED", None)


def test_batchnorm_large_mean_and_zero_variance(T):
    """Statistics stay accurate when |mean| >> sigma; invStd = 0 for a constant channel with eps = 0."""
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(41)
    x = (rng.standard_normal((16, 4, 20, 20)) * 0.01 + 100.0).astype(np.float32)
    trm, trv, tsm, tss, out = (CT.from_numpy(np.zeros(4, np.float32)), CT.from_numpy(np.ones(4, np.float32)),
                               CT.with_size(4), CT.with_size(4), CT())
    THNN.BatchNormalization_updateOutput(CT.from_numpy(x), out, None, None, trm, trv, tsm, tss, True, 0.1, 1e-5)
    rm, rv = np.zeros(4, np.float32), np.ones(4, np.float32)
    ry, sm, ss = O.bn_updateOutput(x, None, None, rm, rv, True, 0.1, 1e-5)
    close(tss.numpy(), ss, WG_RTOL, 0)
    close(tsm.numpy(), sm, 1e-6, 0)
    close(out.numpy(), ry, 1e-3, 2e-3)
    xc = np.full((2, 1, 3), 4.0, np.float32)
    t1, t2, t3, t4 = CT.from_numpy(np.zeros(1, np.float32)), CT.from_numpy(np.ones(1, np.float32)), CT.with_size(1), CT.with_size(1)
    THNN.BatchNormalization_updateOutput(CT.from_numpy(xc), out, None, None, t1, t2, t3, t4, True, 0.1, 0.0)
    assert t4.numpy()[0] == 0 and t3.numpy()[0] == 4 and np.all(out.numpy() == 0)


# --------------------------------------------------------------------- ConvMM --
CONV_CASES = [
    # N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH
    (4, 16, 32, 28, 28, 3, 3, 1, 1, 1, 1),
    (4, 7, 8, 20, 23, 3, 5, 2, 1, 1, 0),
    (8, 32, 64, 14, 14, 3, 3, 1, 1, 1, 1),
    (2, 3, 24, 40, 37, 7, 4, 3, 2, 1, 1),
    (5, 1, 16, 19, 19, 5, 5, 2, 2, 0, 0),
    (3, 130, 136, 9, 9, 3, 3, 1, 1, 1, 1),   # Cout, K not multiples of the GEMM tile
    (2, 8, 200, 16, 16, 1, 1, 1, 1, 0, 0),
    (5, 16, 8, 83, 83, 3, 3, 1, 1, 1, 1),    # more tiles than CUs: the last round is split along K
    (3, 6, 10, 15, 17, 5, 3, 1, 1, 2, 0),    # rectangular kernel, stride 1: gradInput through the forward kernel
    (2, 4, 6, 9, 9, 1, 1, 1, 1, 1, 1),       # pad > k-1: gradInput through gradient columns + col2im
    (2, 8, 12, 70, 70, 3, 3, 1, 1, 1, 1),
]


def _conv_run(T, case, bias=True, weight4d=False, xt=None, scale=1.0, seed=50):
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH = case
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(seed)
    K = Cin * kH * kW
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, K)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32) if bias else None
    tx = xt(x) if xt else CT.from_numpy(x)
    tw = CT.from_numpy(w.reshape(Cout, Cin, kH, kW) if weight4d else w)
    tb = CT.from_numpy(b) if bias else None
    out, cols, ones = CT(), CT(), CT()
    THNN.SpatialConvolutionMM_updateOutput(tx, out, tw, tb, cols, ones, kW, kH, dW, dH, pW, pH)
    ry = O.convmm_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH)
    assert out.size() == ry.shape
    close(out.numpy(), ry)
    gy = rng.standard_normal(ry.shape).astype(np.float32)
    tgy, gi = CT.from_numpy(gy), CT()
    THNN.SpatialConvolutionMM_updateGradInput(tx, tgy, gi, tw, cols, ones, kW, kH, dW, dH, pW, pH)
    close(gi.numpy(), O.convmm_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH))
    gw0 = rng.standard_normal(w.shape).astype(np.float32) * 0.1
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    tgw = CT.from_numpy(gw0.reshape(Cout, Cin, kH, kW) if weight4d else gw0)
    tgb = CT.from_numpy(gb0) if bias else None
    THNN.SpatialConvolutionMM_accGradParameters(tx, tgy, tgw, tgb, cols, ones, kW, kH, dW, dH, pW, pH, scale)
    rgw, rgb = O.convmm_accGradParameters(x, gy, gw0.copy(), gb0.copy() if bias else None, kW, kH, dW, dH, pW, pH, scale)
    close(tgw.numpy().reshape(Cout, K), rgw, WG_RTOL, 1e-3)
    if bias:
        close(tgb.numpy(), rgb, WG_RTOL, 1e-3)


@pytest.mark.parametrize("case", CONV_CASES)
def test_convmm(T, case):
    _conv_run(T, case)


def test_convmm_first_generation_kernels(T):
    cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", "1")
    try:
        _conv_run(T, CONV_CASES[0])
        _conv_run(T, CONV_CASES[3])
    finally:
        cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", None)


def test_convmm_variants(T):
    rng = np.random.default_rng(51)
    _conv_run(T, CONV_CASES[0], bias=False, weight4d=True, scale=0.5)
    _conv_run(T, CONV_CASES[1], xt=lambda a: T.CudaTensor.noncontiguous_from_numpy(a, rng), scale=2.0)


def test_convmm_single_image(T):
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(52)
    x = rng.standard_normal((6, 12, 13)).astype(np.float32)
    w = rng.standard_normal((10, 6 * 9)).astype(np.float32) * 0.2
    out = CT()
    THNN.SpatialConvolutionMM_updateOutput(CT.from_numpy(x), out, CT.from_numpy(w), None, CT(), CT(), 3, 3, 1, 1, 1, 1)
    assert out.size() == (10, 12, 13)
    close(out.numpy(), O.convmm_updateOutput(x[None], w, None, 3, 3, 1, 1, 1, 1)[0])


def test_im2col_col2im(T):
    """lib/THCUNN/im2col.h semantics (incl. dilation) for the stand-alone kernels."""
    import ctypes as C
    from cunn_amd import _lib
    from cunn_amd.tensor import check, state
    CT = T.CudaTensor
    lib = _lib.load()
    rng = np.random.default_rng(53)
    for (Cc, H, W, kH, kW, pH, pW, dH, dW, dlH, dlW) in [(3, 9, 11, 3, 3, 1, 1, 1, 1, 1, 1), (2, 12, 10, 3, 2, 1, 0, 2, 3, 2, 1),
                                                         (4, 8, 8, 5, 3, 2, 1, 1, 2, 1, 2)]:
        im = rng.standard_normal((2, Cc, H, W)).astype(np.float32)
        ref = np.stack([O.im2col(im[n], kW, kH, dW, dH, pW, pH, dlW, dlH) for n in range(2)])
        tim, tcol = CT.from_numpy(im), CT.with_size(*ref.shape)
        lib.THNN_Cuda_im2col(state(), C.c_void_p(tim.data_ptr()), 2, Cc, H, W, kH, kW, pH, pW, dH, dW, dlH, dlW,
                             C.c_void_p(tcol.data_ptr()))
        check()
        assert np.array_equal(tcol.numpy(), ref)
        col = rng.standard_normal(ref.shape).astype(np.float32)
        rim = np.stack([O.col2im(col[n], Cc, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH) for n in range(2)])
        tcol2, tim2 = CT.from_numpy(col), CT.with_size(2, Cc, H, W)
        lib.THNN_Cuda_col2im(state(), C.c_void_p(tcol2.data_ptr()), 2, Cc, H, W, kH, kW, pH, pW, dH, dW, dlH, dlW,
                             C.c_void_p(tim2.data_ptr()))
        check()
        close(tim2.numpy(), rim, 1e-6, 1e-6)

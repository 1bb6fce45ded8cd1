"""SpatialConvolutionMM + Threshold(0, 0) in one pass (include/THCUNN_fused.h; no counterpart in the reference's C ABI):
the clamp v > 0 ? v : 0 of lib/THCUNN/generic/Threshold.cu:7-35 applied as the convolution of
lib/THCUNN/generic/SpatialConvolutionMM.cu:58-209 stores its values. Checked bit for bit against this library's own
two-call sequence on every forward kernel (pointwise, the three tile shapes, whole and K-split tiles, the
first-generation kernel), and against the oracle's composition at the convolution tolerance (1e-5 rel / 1e-4 abs)."""
import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402

# N, Cin, Cout, H, W, k, stride, pad
CASES = [
    (2, 64, 64, 14, 14, 1, 1, 0),     # pointwise kernel, K = 64
    (2, 128, 128, 14, 14, 1, 1, 0),   # pointwise kernel, K = 128
    (3, 32, 40, 10, 10, 1, 1, 0),     # pointwise kernel, K = 32, ragged rows
    (2, 256, 64, 8, 8, 1, 1, 0),      # tiled kernel, 1x1 window (computed tap offsets), every tile split along K
    (2, 16, 128, 12, 12, 3, 1, 1),    # 128 x 128 tiles
    (2, 16, 64, 12, 12, 3, 1, 1),     # 64 x 256 tiles
    (2, 8, 32, 12, 12, 3, 2, 1),      # 32 x 256 tiles, stride 2
    (2, 3, 24, 20, 20, 5, 1, 2),      # K = 75: weight rows padded to the k-tile
    (4, 64, 64, 28, 28, 3, 1, 1),     # 13 tiles: every tile split along K, folded by the second launch
    (1, 8, 8, 9, 7, 3, 1, 1),         # one image, 3-D input below
]


def _both(x, w, b, g):
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    tx, tw = CT.from_numpy(x), CT.from_numpy(w)
    tb = CT.from_numpy(b) if b is not None else None
    fused, plain, relu = CT(), CT(), CT()
    THNN.SpatialConvolutionMMReLU_updateOutput(tx, fused, tw, tb, CT(), CT(), *g)
    THNN.SpatialConvolutionMM_updateOutput(tx, plain, tw, tb, CT(), CT(), *g)
    THNN.Threshold_updateOutput(plain, relu, 0.0, 0.0, False)
    return fused.numpy(), relu.numpy()


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("bias", [True, False])
@pytest.mark.parametrize("generic", [False, True])
def test_conv_relu_forward(case, bias, generic):
    print("case", case, "bias", bias, "generic", generic, flush=True)
    N, Ci, Co, H, W, k, st, pad = case
    rng = np.random.default_rng(123)
    K = Ci * k * k
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    x[0, :, :2, :] = 0.0                      # windows that sum to exactly zero
    w = (rng.standard_normal((Co, K)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32) if bias else None
    if N == 1:
        x = x[0]
    g = (k, k, st, st, pad, pad)
    cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", "1" if generic else None)
    try:
        fused, two = _both(x, w, b, g)
    finally:
        cunn_amd.set_switch("THCUNN_CONV_FORCE_GENERIC", None)
    assert fused.shape == two.shape
    assert np.array_equal(fused.view(np.uint32), two.view(np.uint32)), "fused and two-call results differ"
    ref = O.threshold_updateOutput(O.convmm_updateOutput(x if x.ndim == 4 else x[None], w, b, *g), 0.0, 0.0)
    np.testing.assert_allclose(fused.reshape(ref.shape), ref, rtol=1e-5, atol=1e-4)
    assert (fused >= 0).all() and (fused == 0).any() and (fused > 0).any()


def test_conv_relu_nan_and_negative_zero():
    """v > 0 ? v : 0: a NaN pre-activation stores 0, as Threshold does."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 16, 10, 10)).astype(np.float32)
    x[1, 3, 4, 5] = np.nan
    w = rng.standard_normal((32, 16 * 9)).astype(np.float32)
    fused, two = _both(x, w, None, (3, 3, 1, 1, 1, 1))
    assert np.array_equal(fused.view(np.uint32), two.view(np.uint32))
    assert not np.isnan(fused).any()

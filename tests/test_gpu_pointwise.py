"""1x1 convolutions with short reductions (Cin = 32 ... 256) run on a weight-stationary, position-streaming
kernel of their own; every launch shape of it, ragged ends included, against the oracle through
SpatialConvolutionMM_updateOutput / _updateGradInput (lib/THCUNN/generic/SpatialConvolutionMM.cu:58-325)."""
import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402

# N, Cin, Cout, H, W
CASES = [
    (2, 32, 64, 12, 12),     # K = 32: 64 rows, the waves pair up along the positions
    (3, 32, 24, 10, 10),     # 32 rows or fewer: the tiled GEMM; 300 positions: images end inside tiles
    (3, 32, 40, 10, 10),     # 64-row shape with 40 rows
    (2, 32, 136, 8, 8),      # 128-row blocks, the second with 8 rows
    (1, 32, 256, 6, 6),      # 256 rows per workgroup; 36 positions: one full tile and one of 4
    (2, 64, 64, 14, 14),     # K = 64
    (2, 64, 128, 14, 14),
    (2, 64, 264, 6, 10),
    (2, 64, 16, 10, 10),
    (2, 128, 128, 14, 14),   # K = 128
    (3, 128, 48, 10, 10),
    (2, 128, 256, 8, 8),     # two row blocks of 128
    (2, 128, 24, 8, 8),      # the tiled GEMM
    (2, 256, 64, 8, 8),      # K = 256: the tiled GEMM
    (2, 256, 128, 14, 14),
    (1, 256, 512, 6, 6),
    (5, 128, 128, 28, 28),   # 3920 positions: 123 tiles
    (1, 64, 64, 4, 8),       # a single tile
]


def _run(case, bias=True, seed=70, cap=None):
    N, Ci, Co, H, W = case
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci)) * np.sqrt(2.0 / Ci)).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32) if bias else None
    gy = rng.standard_normal((N, Co, H, W)).astype(np.float32)
    g = (1, 1, 1, 1, 0, 0)
    ry = O.convmm_updateOutput(x, w, b, *g)
    rgx = O.convmm_updateGradInput(x.shape, gy, w, *g)
    tx, tw, tgy = CT.from_numpy(x), CT.from_numpy(w), CT.from_numpy(gy)
    tb = CT.from_numpy(b) if bias else None
    results = {}
    for mode in ([cap] if cap else []) + [None, "0"]:   # the streaming kernel (few workgroups / default), then the tiled GEMM
        cunn_amd.set_switch("THCUNN_CONV_POINTWISE", mode)
        try:
            out, gx = CT(), CT()
            THNN.SpatialConvolutionMM_updateOutput(tx, out, tw, tb, CT(), CT(), *g)
            THNN.SpatialConvolutionMM_updateGradInput(tx, tgy, gx, tw, CT(), CT(), *g)
            yv, gxv = out.numpy(), gx.numpy()
        finally:
            cunn_amd.set_switch("THCUNN_CONV_POINTWISE", None)
        assert yv.shape == ry.shape
        np.testing.assert_allclose(yv, ry, rtol=1e-5, atol=1e-4, err_msg=f"updateOutput, switch {mode}")
        np.testing.assert_allclose(gxv, rgx, rtol=1e-5, atol=1e-4, err_msg=f"updateGradInput, switch {mode}")
        results[mode] = (yv, gxv)
    if cap:   # the result does not depend on how the positions are dealt to workgroups
        assert np.array_equal(results[cap][0], results[None][0]) and np.array_equal(results[cap][1], results[None][1])


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("bias", [True, False])
def test_pointwise_convolution(case, bias):
    print("case", case, "bias", bias, flush=True)
    _run(case, bias)


@pytest.mark.parametrize("case", [(5, 128, 128, 28, 28), (4, 64, 128, 20, 20), (6, 32, 64, 18, 18), (3, 256, 128, 20, 20),
                                  (4, 64, 320, 12, 12)])
@pytest.mark.parametrize("cap", ["2", "3", "7"])
def test_pointwise_long_runs_of_tiles(case, cap):
    """Few workgroups: each streams many chunks (the steady state of the pipeline) and ends on a partial one."""
    print("case", case, "cap", cap, flush=True)
    _run(case, True, seed=71, cap=cap)


def test_pointwise_mobilenet_layer_full_size():
    """128 -> 128 at 56 x 56, N = 64 (the pointwise layer behind the benchmark's depthwise layer)."""
    _run((64, 128, 128, 56, 56), True, seed=72)

"""Tile shapes of the SpatialConvolutionMM kernels (lib/THCUNN/generic/SpatialConvolutionMM.cu:58-486): the forward
pass and the stride-1 gradInput have 128 x 128, 64 x 256 and 32 x 256 output tiles, the weight gradient large tiles
and small ones of 1x1, 1x2, 1x4, 2x1 or 2x2 blocks of 32 x 32; the shape follows from Cout, Cin and K = Cin kH kW.
One case per shape (ragged rows and columns included), and the K-splits the planner picks for grids that do not
fill the CUs evenly, against the oracle."""
import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402

# N, Cin, Cout, H, W, k, stride, pad; gradWeight is Cout x (Cin k k)
CASES = [
    (2, 3, 32, 20, 20, 3, 2, 1),     # gradWeight 32 x 27: one 32 x 32 tile; forward: 32 rows
    (2, 3, 30, 21, 19, 3, 1, 1),     # 30 x 27, ragged
    (2, 32, 32, 18, 18, 3, 1, 0),    # 32 x 288: 32 x 64 tiles; gradInput on 32 rows
    (2, 24, 24, 16, 16, 3, 1, 1),    # 24 x 216: 32 x 128 tiles
    (2, 3, 64, 20, 20, 3, 1, 1),     # 64 x 27: 64 x 32 tiles
    (2, 3, 64, 30, 30, 7, 2, 3),     # 64 x 147: 64 x 32 tiles, five of them
    (2, 32, 64, 16, 16, 3, 1, 1),    # 64 x 288: 64 x 64 tiles; gradInput with 32 rows
    (2, 64, 80, 12, 12, 1, 1, 0),    # 80 x 64: 32 x 64 tiles, three row tiles; forward: 3 tiles of 32 rows (80 = 64 + 16)
    (2, 64, 96, 10, 10, 3, 1, 1),    # forward: 96 rows as three 32-row tiles; gradWeight on large tiles
    (3, 256, 21, 12, 12, 1, 1, 0),   # 21 rows
    (2, 16, 16, 24, 24, 3, 1, 1),
    (2, 64, 32, 14, 14, 1, 1, 0),    # gradWeight 32 x 64
    (4, 64, 64, 28, 28, 3, 1, 1),    # 13 tiles of 64 x 256: every tile split along K
    (9, 128, 128, 14, 14, 3, 1, 1),  # 14 tiles of 128 x 128
    (2, 64, 128, 16, 16, 1, 2, 0),   # 1x1 stride 2, even extents: gradInput written as 2 x 2 blocks by one pointwise pass
    (3, 20, 24, 10, 14, 1, 2, 0),    # the same with 20 rows (element-wise stores) and K = 24
    (2, 40, 256, 8, 12, 1, 2, 0),    # 40 rows: a full 32-row tile and a partial one
    (2, 256, 64, 8, 8, 1, 2, 0),     # every tile split along K: the blocks are written by the fold
    (2, 64, 128, 15, 17, 1, 2, 0),   # odd extents: phase by phase
    # weight gradient on large tiles with the image gathered 16 bytes at a time (unit stride; 4 positions inside a row)
    (2, 32, 128, 12, 12, 3, 1, 1),   # 128 x 128 tiles, rows of 12, every k-tile inside one image
    (2, 40, 130, 8, 16, 3, 1, 1),    # ragged rows and columns, unaligned groups
    (2, 64, 64, 12, 12, 3, 1, 1),    # 64 x 256 tiles
    (4, 128, 128, 14, 14, 1, 1, 0),  # rows of 14: groups straddle rows that follow each other without a gap (1x1, no padding)
    (3, 128, 128, 14, 12, 3, 1, 0),  # output rows of 10: element-wise gather
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("bias", [True, False])
def test_conv_tile_shapes(case, bias):
    print("case", case, "bias", bias, flush=True)
    N, Ci, Co, H, W, k, st, pad = case
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(90)
    K = Ci * k * k
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Co, K)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32) if bias else None
    g = (k, k, st, st, pad, pad)
    ry = O.convmm_updateOutput(x, w, b, *g)
    gy = rng.standard_normal(ry.shape).astype(np.float32)
    rgx = O.convmm_updateGradInput(x.shape, gy, w, *g)
    gw0 = rng.standard_normal((Co, K)).astype(np.float32)
    gb0 = rng.standard_normal(Co).astype(np.float32)
    rgw, rgb = O.convmm_accGradParameters(x, gy, gw0.copy(), gb0.copy() if bias else None, *g, 0.5)
    tx, tw, tgy = CT.from_numpy(x), CT.from_numpy(w), CT.from_numpy(gy)
    tb = CT.from_numpy(b) if bias else None
    out, gx = CT(), CT()
    THNN.SpatialConvolutionMM_updateOutput(tx, out, tw, tb, CT(), CT(), *g)
    THNN.SpatialConvolutionMM_updateGradInput(tx, tgy, gx, tw, CT(), CT(), *g)
    tgw = CT.from_numpy(gw0)
    tgb = CT.from_numpy(gb0) if bias else None
    THNN.SpatialConvolutionMM_accGradParameters(tx, tgy, tgw, tgb, CT(), CT(), *g, 0.5)
    np.testing.assert_allclose(out.numpy(), ry, rtol=1e-5, atol=1e-4, err_msg="updateOutput")
    np.testing.assert_allclose(gx.numpy(), rgx, rtol=1e-5, atol=1e-4, err_msg="updateGradInput")
    # sums over N * L positions in another order than the oracle's: the weight-gradient bound
    np.testing.assert_allclose(tgw.numpy(), rgw, rtol=1e-3, atol=1e-3, err_msg="gradWeight")
    if bias:
        np.testing.assert_allclose(tgb.numpy(), rgb, rtol=1e-3, atol=1e-3, err_msg="gradBias")


@pytest.mark.parametrize("case", [(2, 96, 48, 9, 11), (3, 16, 20, 6, 6), (2, 128, 256, 7, 7)])
@pytest.mark.parametrize("bias", [True, False])
def test_transposed_1x1_stride2_forward(case, bias):
    """SpatialFullConvolution (lib/THCUNN/generic/SpatialFullDilatedConvolution.cu:141-165) with a 1x1 window, stride 2 and
    output padding 1: every input element lands on the top-left corner of a 2 x 2 output block, the rest is the bias."""
    print("case", case, "bias", bias, flush=True)
    N, Ci, Co, H, W = case
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(91)
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Ci, Co, 1, 1)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32) if bias else None
    g = (1, 1, 2, 2, 0, 0, 1, 1)
    ref = O.fullconv_updateOutput(x, w, b, 1, 1, 2, 2, 0, 0, adjW=1, adjH=1)
    out = CT()
    THNN.SpatialFullConvolution_updateOutput(CT.from_numpy(x), out, CT.from_numpy(w), CT.from_numpy(b) if bias else None,
                                             CT(), CT(), *g)
    got = out.numpy()
    assert got.shape == ref.shape == (N, Co, 2 * H, 2 * W)
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-4)

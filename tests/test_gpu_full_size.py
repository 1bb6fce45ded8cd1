"""The five benchmark configurations at their full sizes on the GPU: compared with
the CPU oracle where it finishes in seconds, and through size-independent
properties (adjoint identities, index round trips, gradient orthogonality)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402


@pytest.fixture(scope="module")
def T():
    import cunn_amd
    return cunn_amd


def dot(a, b):
    return float(np.vdot(a.astype(np.float64), b.astype(np.float64)))


def test_cfg1_depthwise_forward(T):
    CT, THNN = T.CudaTensor, T.THNN
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, (32, 32, 112, 112)).astype(np.float32)
    b9 = np.sqrt(6.0 / 9)
    w = rng.uniform(-b9, b9, (1, 32, 3, 3)).astype(np.float32)
    b = rng.uniform(-1 / 3, 1 / 3, (1, 32)).astype(np.float32)
    y = CT()
    THNN.SpatialDepthWiseConvolution_updateOutput(CT.from_numpy(x), y, CT.from_numpy(w), CT.from_numpy(b), CT(), CT(), 3, 3, 1, 1, 1, 1)
    np.testing.assert_allclose(y.numpy(), O.dwconv_updateOutput(x, w, b, 3, 3, 1, 1, 1, 1), rtol=1e-5, atol=1e-4)


def test_cfg2_depthwise_fwd_bwd(T):
    CT, THNN = T.CudaTensor, T.THNN
    rng = np.random.default_rng(1)
    N, C, H = 64, 128, 56
    x = rng.standard_normal((N, C, H, H)).astype(np.float32)
    gy = rng.standard_normal((N, C, 28, 28)).astype(np.float32)
    b9 = np.sqrt(6.0 / 9)
    w = rng.uniform(-b9, b9, (1, C, 3, 3)).astype(np.float32)
    g = (3, 3, 2, 2, 1, 1)
    tx, tgy, tw = CT.from_numpy(x), CT.from_numpy(gy), CT.from_numpy(w)
    y, gx, cols, ones = CT(), CT(), CT(), CT()
    THNN.SpatialDepthWiseConvolution_updateOutput(tx, y, tw, None, cols, ones, *g)
    THNN.SpatialDepthWiseConvolution_updateGradInput(tx, tgy, gx, tw, cols, ones, *g)
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    tgw = CT.from_numpy(gw0)
    THNN.SpatialDepthWiseConvolution_accGradParameters(tx, tgy, tgw, None, cols, ones, *g, 1.0)
    yv, gxv, gwv = y.numpy(), gx.numpy(), tgw.numpy()
    np.testing.assert_allclose(yv, O.dwconv_updateOutput(x, w, None, *g), rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(gxv, O.dwconv_updateGradInput(x.shape, gy, w, *g), rtol=1e-5, atol=1e-4)
    rgw, _ = O.dwconv_accGradParameters(x, gy, gw0.copy(), None, *g, 1.0)
    np.testing.assert_allclose(gwv, rgw, rtol=1e-3, atol=1e-2)   # accumulates into non-zero values
    # adjoint identity: <DW(x), gy> = <x, gradInput(gy)> = <w, gradW - gradW0>
    lhs = dot(yv, gy)
    assert abs(lhs - dot(x, gxv)) <= 1e-5 * abs(lhs) + 1.0
    assert abs(lhs - dot(w, gwv - gw0)) <= 1e-4 * abs(lhs) + 1.0


def test_cfg3_batchnorm_train(T):
    CT, THNN = T.CudaTensor, T.THNN
    rng = np.random.default_rng(2)
    N, C, H = 64, 256, 28
    x = (rng.standard_normal((N, C, H, H)) * 2 + 0.5).astype(np.float32)
    gy = rng.standard_normal((N, C, H, H)).astype(np.float32)
    g = rng.random(C).astype(np.float32)
    b = rng.standard_normal(C).astype(np.float32)
    tx, tgy, tg, tb = CT.from_numpy(x), CT.from_numpy(gy), CT.from_numpy(g), CT.from_numpy(b)
    rm, rv, sm, ss = CT.from_numpy(np.zeros(C, np.float32)), CT.from_numpy(np.ones(C, np.float32)), CT.with_size(C), CT.with_size(C)
    y, gx = CT(), CT.with_size(N, C, H, H)
    gw, gb = CT.from_numpy(np.zeros(C, np.float32)), CT.from_numpy(np.zeros(C, np.float32))
    THNN.BatchNormalization_updateOutput(tx, y, tg, tb, rm, rv, sm, ss, True, 0.1, 1e-5)
    THNN.BatchNormalization_backward(tx, tgy, gx, gw, gb, tg, rm, rv, sm, ss, True, 1.0, 1e-5)
    orm, orv = np.zeros(C, np.float32), np.ones(C, np.float32)
    ry, osm, oss = O.bn_updateOutput(x, g, b, orm, orv, True, 0.1, 1e-5)
    np.testing.assert_allclose(y.numpy(), ry, rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(sm.numpy(), osm, rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(ss.numpy(), oss, rtol=1e-3)
    np.testing.assert_allclose(rm.numpy(), orm, rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(rv.numpy(), orv, rtol=1e-3)
    rgx, rgw, rgb = O.bn_backward(x, gy, g, orm, orv, osm, oss, True, 1.0, 1e-5, np.zeros(C, np.float32), np.zeros(C, np.float32))
    gxv = gx.numpy()
    np.testing.assert_allclose(gxv, rgx, rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(gw.numpy(), rgw, rtol=1e-3, atol=5e-2)
    np.testing.assert_allclose(gb.numpy(), rgb, rtol=1e-3, atol=5e-2)
    # per channel: output mean = beta, output variance = gamma^2 var/(var+eps); gradInput sums to zero
    yv = y.numpy().astype(np.float64)
    np.testing.assert_allclose(yv.mean(axis=(0, 2, 3)), b, atol=1e-4)
    assert np.all(np.abs(gxv.astype(np.float64).sum(axis=(0, 2, 3))) < 5e-2)


def test_cfg4_pooling(T):
    CT, LT, THNN = T.CudaTensor, T.CudaLongTensor, T.THNN
    rng = np.random.default_rng(3)
    N, C, H = 64, 64, 112
    x = (np.round(rng.uniform(-1, 1, (N, C, H, H)) * 64) / 64).astype(np.float32)
    gy = rng.standard_normal((N, C, 56, 56)).astype(np.float32)
    tx, tgy = CT.from_numpy(x), CT.from_numpy(gy)
    y, idx, gx, ya, gxa = CT(), LT(), CT(), CT(), CT()
    THNN.SpatialMaxPooling_updateOutput(tx, y, idx, 3, 3, 2, 2, 1, 1, False)
    THNN.SpatialMaxPooling_updateGradInput(tx, tgy, gx, idx, 3, 3, 2, 2, 1, 1, False)
    THNN.SpatialAveragePooling_updateOutput(tx, ya, 2, 2, 2, 2, 0, 0, False, True)
    THNN.SpatialAveragePooling_updateGradInput(tx, tgy, gxa, 2, 2, 2, 2, 0, 0, False, True)
    ry, ridx = O.maxpool_updateOutput(x, 3, 3, 2, 2, 1, 1, False)
    yv, iv = y.numpy(), idx.numpy()
    assert np.array_equal(yv, ry) and np.array_equal(iv, ridx)
    # index round trip and gradient mass conservation
    flat = x.reshape(N, C, -1)
    assert np.array_equal(np.take_along_axis(flat, (iv - 1).reshape(N, C, -1), axis=2).reshape(yv.shape), yv)
    gxv = gx.numpy()
    np.testing.assert_allclose(gxv, O.maxpool_updateGradInput(x.shape, gy, ridx, 3, 3, 2, 2, 1, 1, False), rtol=1e-5, atol=1e-4)
    assert abs(gxv.astype(np.float64).sum() - gy.astype(np.float64).sum()) < 1.0
    np.testing.assert_allclose(ya.numpy(), O.avgpool_updateOutput(x, 2, 2, 2, 2, 0, 0, False, True), rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(gxa.numpy(), O.avgpool_updateGradInput(x.shape, gy, 2, 2, 2, 2, 0, 0, False, True), rtol=1e-5, atol=1e-4)


def test_cfg5_convmm(T):
    CT, THNN = T.CudaTensor, T.THNN
    rng = np.random.default_rng(4)
    N, Ci, Co, H = 64, 256, 256, 28
    K = Ci * 9
    x = rng.standard_normal((N, Ci, H, H)).astype(np.float32)
    gy = rng.standard_normal((N, Co, H, H)).astype(np.float32)
    w = (rng.standard_normal((Co, K)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.uniform(-0.02, 0.02, Co).astype(np.float32)
    g = (3, 3, 1, 1, 1, 1)
    tx, tgy, tw, tb = CT.from_numpy(x), CT.from_numpy(gy), CT.from_numpy(w), CT.from_numpy(b)
    y, gx, cols, gcols, ones = CT(), CT(), CT(), CT(), CT()
    gw, gb = CT.from_numpy(np.zeros_like(w)), CT.from_numpy(np.zeros_like(b))
    THNN.SpatialConvolutionMM_updateOutput(tx, y, tw, tb, cols, ones, *g)
    THNN.SpatialConvolutionMM_updateGradInput(tx, tgy, gx, tw, gcols, ones, *g)
    THNN.SpatialConvolutionMM_accGradParameters(tx, tgy, gw, gb, cols, ones, *g, 1.0)
    yv, gxv, gwv, gbv = y.numpy(), gx.numpy(), gw.numpy(), gb.numpy()
    m = [0, 31, 63]                                     # images checked against the oracle
    np.testing.assert_allclose(yv[m], O.convmm_updateOutput(x[m], w, b, *g), rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(gxv[m], O.convmm_updateGradInput((len(m),) + x.shape[1:], gy[m], w, *g), rtol=1e-5, atol=1e-4)
    np.testing.assert_allclose(gbv, gy.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-3, atol=5e-2)
    # adjoint identities over the whole batch: <conv(x) - b, gy> = <x, gradInput> = <W, gradW>
    lhs = dot(yv - b[None, :, None, None], gy)
    assert abs(lhs - dot(x, gxv)) <= 1e-4 * abs(lhs) + 5.0
    assert abs(lhs - dot(w, gwv)) <= 1e-4 * abs(lhs) + 5.0
    # gradWeight of the whole batch (the call that plans the many-way position split, its partial tiles and their
    # fold), element by element against the same sum in float64: per image the im2col matrix as a strided view of
    # the zero-padded image (2304 x 784) times gradOutput (256 x 784) transposed, 59 GFLOP of float64 BLAS
    ref = np.zeros((Co, K))
    xp = np.zeros((Ci, H + 2, H + 2))
    for n in range(N):
        xp[:, 1:-1, 1:-1] = x[n]
        win = np.lib.stride_tricks.sliding_window_view(xp, (3, 3), axis=(1, 2))      # (Ci, H, H, 3, 3)
        col = win.transpose(0, 3, 4, 1, 2).reshape(K, H * H)                        # row (c, kh, kw), column (oh, ow)
        ref += gy[n].reshape(Co, H * H).astype(np.float64) @ col.T
    np.testing.assert_allclose(gwv, ref, rtol=1e-3, atol=0.05)   # values are +-224 (50 176 terms of unit variance)
    # gradWeight against the oracle on the first four images (the full batch takes the CPU minutes)
    sub = slice(0, 4)
    gws = CT.from_numpy(np.zeros_like(w))
    THNN.SpatialConvolutionMM_accGradParameters(CT.from_numpy(x[sub]), CT.from_numpy(gy[sub]), gws, None, cols, ones, *g, 1.0)
    rgw, _ = O.convmm_accGradParameters(x[sub], gy[sub], np.zeros_like(w), None, *g, 1.0)
    np.testing.assert_allclose(gws.numpy(), rgw, rtol=1e-3, atol=2e-3)

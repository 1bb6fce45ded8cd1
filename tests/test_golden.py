"""Committed golden vectors (tests/golden/thnn_golden.npz, written by
tests/golden/make_golden.py from PyTorch-CPU float64 operators and the
reference's literal known answers) against both implementations:
the CPU oracle (runs everywhere) and the HIP library through the C ABI (GPU)."""
import os

import numpy as np
import pytest

from oracle import oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "thnn_golden.npz"))


def case(name):
    return {k.split("/", 1)[1]: G[k] for k in G.files if k.startswith(name + "/")}


def close(a, b, rtol=1e-5, atol=1e-4):
    np.testing.assert_allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), rtol=rtol, atol=atol)


class OracleBackend:
    name = "oracle"

    def dw(self, c):
        g = [int(v) for v in c["geom"]]
        y = O.dwconv_updateOutput(c["x"], c["w"], c["b"], *g)
        gx = O.dwconv_updateGradInput(c["x"].shape, c["gy"], c["w"], *g)
        gw, gb = O.dwconv_accGradParameters(c["x"], c["gy"], np.zeros_like(c["w"]), np.zeros_like(c["b"]), *g, 1.0)
        return y, gx, gw, gb

    def conv(self, c):
        g = [int(v) for v in c["geom"]]
        y = O.convmm_updateOutput(c["x"], c["w"], c["b"], *g)
        gx = O.convmm_updateGradInput(c["x"].shape, c["gy"], c["w"], *g)
        gw, gb = O.convmm_accGradParameters(c["x"], c["gy"], np.zeros_like(c["w"]), np.zeros_like(c["b"]), *g, 1.0)
        return y, gx, gw, gb

    def bn(self, c):
        C = c["g"].shape[0]
        rm, rv = np.zeros(C, np.float32), np.ones(C, np.float32)
        y, sm, ss = O.bn_updateOutput(c["x"], c["g"], c["b"], rm, rv, True, 0.1, 1e-5)
        gx, gw, gb = O.bn_backward(c["x"], c["gy"], c["g"], rm, rv, sm, ss, True, 1.0, 1e-5,
                                   np.zeros(C, np.float32), np.zeros(C, np.float32))
        ye, _, _ = O.bn_updateOutput(c["x"], c["g"], c["b"], rm.copy(), rv.copy(), False, 0.1, 1e-5)
        return y, sm, ss, rm, rv, gx, gw, gb, ye

    def maxpool(self, c):
        k, _, s, _, p, _, ceil = [int(v) for v in c["geom"]]
        y, idx = O.maxpool_updateOutput(c["x"], k, k, s, s, p, p, bool(ceil))
        gx = O.maxpool_updateGradInput(c["x"].shape, c["gy"], idx, k, k, s, s, p, p, bool(ceil))
        return y, idx, gx

    def avgpool(self, c, inc, x=None):
        k, _, s, _, p, _, ceil = [int(v) for v in c["geom"]] if "geom" in c else (2, 2, 1, 1, 1, 1, 0)
        x = c["x"] if x is None else x
        y = O.avgpool_updateOutput(x, k, k, s, s, p, p, bool(ceil), inc)
        gx = O.avgpool_updateGradInput(x.shape, c["gy"], k, k, s, s, p, p, bool(ceil), inc) if "gy" in c else None
        return y, gx


class HipBackend:
    name = "hip"

    def __init__(self):
        import cunn_amd
        self.T = cunn_amd

    def dw(self, c):
        CT, THNN = self.T.CudaTensor, self.T.THNN
        g = [int(v) for v in c["geom"]]
        x, w, b, gy = (CT.from_numpy(c[k]) for k in ("x", "w", "b", "gy"))
        y, gx, cols, ones = CT(), CT(), CT(), CT()
        gw, gb = CT.from_numpy(np.zeros_like(c["w"])), CT.from_numpy(np.zeros_like(c["b"]))
        THNN.SpatialDepthWiseConvolution_updateOutput(x, y, w, b, cols, ones, *g)
        THNN.SpatialDepthWiseConvolution_updateGradInput(x, gy, gx, w, cols, ones, *g)
        THNN.SpatialDepthWiseConvolution_accGradParameters(x, gy, gw, gb, cols, ones, *g, 1.0)
        return y.numpy(), gx.numpy(), gw.numpy(), gb.numpy()

    def conv(self, c):
        CT, THNN = self.T.CudaTensor, self.T.THNN
        g = [int(v) for v in c["geom"]]
        x, w, b, gy = (CT.from_numpy(c[k]) for k in ("x", "w", "b", "gy"))
        y, gx, cols, ones = CT(), CT(), CT(), CT()
        gw, gb = CT.from_numpy(np.zeros_like(c["w"])), CT.from_numpy(np.zeros_like(c["b"]))
        THNN.SpatialConvolutionMM_updateOutput(x, y, w, b, cols, ones, *g)
        THNN.SpatialConvolutionMM_updateGradInput(x, gy, gx, w, cols, ones, *g)
        THNN.SpatialConvolutionMM_accGradParameters(x, gy, gw, gb, cols, ones, *g, 1.0)
        return y.numpy(), gx.numpy(), gw.numpy(), gb.numpy()

    def bn(self, c):
        CT, THNN = self.T.CudaTensor, self.T.THNN
        C = c["g"].shape[0]
        x, g, b, gy = (CT.from_numpy(c[k]) for k in ("x", "g", "b", "gy"))
        rm, rv = CT.from_numpy(np.zeros(C, np.float32)), CT.from_numpy(np.ones(C, np.float32))
        sm, ss, y, ye = CT.with_size(C), CT.with_size(C), CT(), CT()
        THNN.BatchNormalization_updateOutput(x, y, g, b, rm, rv, sm, ss, True, 0.1, 1e-5)
        gx = CT.with_size(*c["x"].shape)
        gw, gb = CT.from_numpy(np.zeros(C, np.float32)), CT.from_numpy(np.zeros(C, np.float32))
        THNN.BatchNormalization_backward(x, gy, gx, gw, gb, g, rm, rv, sm, ss, True, 1.0, 1e-5)
        THNN.BatchNormalization_updateOutput(x, ye, g, b, rm, rv, sm, ss, False, 0.1, 1e-5)
        return (y.numpy(), sm.numpy(), ss.numpy(), rm.numpy(), rv.numpy(), gx.numpy(), gw.numpy(), gb.numpy(), ye.numpy())

    def maxpool(self, c):
        CT, LT, THNN = self.T.CudaTensor, self.T.CudaLongTensor, self.T.THNN
        k, _, s, _, p, _, ceil = [int(v) for v in c["geom"]]
        x, gy, y, idx, gx = CT.from_numpy(c["x"]), CT.from_numpy(c["gy"]), CT(), LT(), CT()
        THNN.SpatialMaxPooling_updateOutput(x, y, idx, k, k, s, s, p, p, bool(ceil))
        THNN.SpatialMaxPooling_updateGradInput(x, gy, gx, idx, k, k, s, s, p, p, bool(ceil))
        return y.numpy(), idx.numpy(), gx.numpy()

    def avgpool(self, c, inc, x=None):
        CT, THNN = self.T.CudaTensor, self.T.THNN
        k, _, s, _, p, _, ceil = [int(v) for v in c["geom"]] if "geom" in c else (2, 2, 1, 1, 1, 1, 0)
        xa = c["x"] if x is None else x
        tx, y = CT.from_numpy(xa), CT()
        THNN.SpatialAveragePooling_updateOutput(tx, y, k, k, s, s, p, p, bool(ceil), inc)
        gx = None
        if "gy" in c:
            t = CT()
            THNN.SpatialAveragePooling_updateGradInput(tx, CT.from_numpy(c["gy"]), t, k, k, s, s, p, p, bool(ceil), inc)
            gx = t.numpy()
        return y.numpy(), gx


@pytest.fixture(params=["oracle", pytest.param("hip", marks=pytest.mark.gpu)])
def backend(request):
    return OracleBackend() if request.param == "oracle" else HipBackend()


@pytest.mark.parametrize("name", ["dw_ref_shape", "dw_s2", "dw_k5"])
def test_depthwise_golden(backend, name):
    c = case(name)
    y, gx, gw, gb = backend.dw(c)
    close(y, c["y"]); close(gx, c["gx"]); close(gw, c["gw"], 1e-3, 1e-3); close(gb, c["gb"], 1e-3, 1e-3)


@pytest.mark.parametrize("name", ["conv_3x3", "conv_s2"])
def test_convmm_golden(backend, name):
    c = case(name)
    y, gx, gw, gb = backend.conv(c)
    close(y, c["y"]); close(gx, c["gx"]); close(gw, c["gw"], 1e-3, 1e-3); close(gb, c["gb"], 1e-3, 1e-3)


@pytest.mark.parametrize("name", ["bn_4d", "bn_2d"])
def test_batchnorm_golden(backend, name):
    c = case(name)
    y, sm, ss, rm, rv, gx, gw, gb, ye = backend.bn(c)
    close(y, c["y"], 1e-5, 1e-4); close(ye, c["y_eval"], 1e-5, 1e-4)
    close(sm, c["save_mean"], 1e-3, 1e-5); close(ss, c["save_std"], 1e-3, 1e-6)
    close(rm, c["run_mean"], 1e-3, 1e-5); close(rv, c["run_var"], 1e-3, 1e-5)
    close(gx, c["gx"], 1e-5, 1e-4); close(gw, c["gw"], 1e-3, 1e-3); close(gb, c["gb"], 1e-3, 1e-3)


@pytest.mark.parametrize("name", ["pool_3s2p1", "pool_2s2", "pool_3s2p1_ceil", "pool_2s2p1_ceil_drop"])
def test_pooling_golden(backend, name):
    c = case(name)
    y, idx, gx = backend.maxpool(c)
    assert np.array_equal(y, c["max_y"]) and np.array_equal(idx, c["max_idx"])   # bit-exact
    close(gx, c["max_gx"])
    for inc in (True, False):
        ya, gxa = backend.avgpool(c, inc)
        close(ya, c[f"avg_y_{int(inc)}"]); close(gxa, c[f"avg_gx_{int(inc)}"])


def test_avgpool_reference_known_answer(backend):
    c = case("kat_avgpool")
    inc, _ = backend.avgpool({}, True, x=c["x"])
    exc, _ = backend.avgpool({}, False, x=c["x"])
    assert exc[0, 0, 0, 0] == c["exclude_pad"] == 3.0
    assert inc[0, 0, 0, 0] == c["include_pad"] == 0.75


# ---- vectors for the entry points next to the hot path: dilated max pooling, dilated and transposed convolution,
# Threshold, and the fused BatchNormalization + ReLU pair ----------------------------------------------------------

def _hip():
    import cunn_amd
    return cunn_amd.CudaTensor, cunn_amd.CudaLongTensor, cunn_amd.THNN


def test_dilated_maxpool_golden(backend):
    c = case("pool_dil2")
    k, _, s, _, p, _, dil, _, ceil = [int(v) for v in c["geom"]]
    if backend.name == "oracle":
        y, idx = O.maxpool_updateOutput(c["x"], k, k, s, s, p, p, bool(ceil), dil, dil)
        gx = O.maxpool_updateGradInput(c["x"].shape, c["gy"], idx, k, k, s, s, p, p, bool(ceil), dil, dil)
    else:
        CT, LT, THNN = _hip()
        x, gy, ty, tidx, tgx = CT.from_numpy(c["x"]), CT.from_numpy(c["gy"]), CT(), LT(), CT()
        THNN.SpatialDilatedMaxPooling_updateOutput(x, ty, tidx, k, k, s, s, p, p, dil, dil, bool(ceil))
        THNN.SpatialDilatedMaxPooling_updateGradInput(x, gy, tgx, tidx, k, k, s, s, p, p, dil, dil, bool(ceil))
        y, idx, gx = ty.numpy(), tidx.numpy(), tgx.numpy()
    assert np.array_equal(y, c["max_y"]) and np.array_equal(idx, c["max_idx"])   # bit-exact
    close(gx, c["max_gx"])


def test_dilated_convolution_golden(backend):
    c = case("dilconv_d2")
    g = [int(v) for v in c["geom"]]
    Co, K = c["w"].shape[0], int(np.prod(c["w"].shape[1:]))
    if backend.name == "oracle":
        y = O.dilconv_updateOutput(c["x"], c["w"], c["b"], *g)
        gx = O.dilconv_updateGradInput(c["x"].shape, c["gy"], c["w"], *g)
        gw, gb = O.dilconv_accGradParameters(c["x"], c["gy"], np.zeros((Co, K), np.float32), np.zeros_like(c["b"]), *g, 1.0)
    else:
        CT, _, THNN = _hip()
        x, w, b, gy = (CT.from_numpy(c[k]) for k in ("x", "w", "b", "gy"))
        ty, tgx, cols, gcols, ones = CT(), CT(), CT(), CT(), CT()
        tgw, tgb = CT.from_numpy(np.zeros_like(c["w"])), CT.from_numpy(np.zeros_like(c["b"]))
        THNN.SpatialDilatedConvolution_updateOutput(x, ty, w, b, cols, ones, *g)
        THNN.SpatialDilatedConvolution_updateGradInput(x, gy, tgx, w, gcols, *g)
        THNN.SpatialDilatedConvolution_accGradParameters(x, gy, tgw, tgb, cols, ones, *g, 1.0)
        y, gx, gw, gb = ty.numpy(), tgx.numpy(), tgw.numpy(), tgb.numpy()
    close(y, c["y"]); close(gx, c["gx"])
    close(np.asarray(gw).reshape(c["gw"].shape), c["gw"], 1e-3, 1e-3); close(gb, c["gb"], 1e-3, 1e-3)


def test_transposed_convolution_golden(backend):
    c = case("fullconv_s2")
    k, _, s, _, p, _, adj, _ = [int(v) for v in c["geom"]]
    if backend.name == "oracle":
        og = (k, k, s, s, p, p, 1, 1, adj, adj)
        y = O.fullconv_updateOutput(c["x"], c["w"], c["b"], *og)
        gx = O.fullconv_updateGradInput(c["x"].shape, c["gy"], c["w"], *og)
        gw, gb = O.fullconv_accGradParameters(c["x"], c["gy"], np.zeros_like(c["w"]), np.zeros_like(c["b"]), *og, scale=1.0)
    else:
        CT, _, THNN = _hip()
        g = (k, k, s, s, p, p, adj, adj)
        x, w, b, gy = (CT.from_numpy(c[n]) for n in ("x", "w", "b", "gy"))
        ty, tgx, cols, gcols, ones = CT(), CT(), CT(), CT(), CT()
        tgw, tgb = CT.from_numpy(np.zeros_like(c["w"])), CT.from_numpy(np.zeros_like(c["b"]))
        THNN.SpatialFullConvolution_updateOutput(x, ty, w, b, cols, ones, *g)
        THNN.SpatialFullConvolution_updateGradInput(x, gy, tgx, w, gcols, *g)
        THNN.SpatialFullConvolution_accGradParameters(x, gy, tgw, tgb, cols, ones, *g, 1.0)
        y, gx, gw, gb = ty.numpy(), tgx.numpy(), tgw.numpy(), tgb.numpy()
    close(y, c["y"]); close(gx, c["gx"])
    close(np.asarray(gw).reshape(c["gw"].shape), c["gw"], 1e-3, 1e-3); close(gb, c["gb"], 1e-3, 1e-3)


def test_threshold_golden(backend):
    c = case("thr")
    th, val = float(c["param"][0]), float(c["param"][1])
    if backend.name == "oracle":
        y, gx = O.threshold_updateOutput(c["x"], th, val), O.threshold_updateGradInput(c["x"], c["gy"], th)
    else:
        CT, _, THNN = _hip()
        x, gy, ty, tgx = CT.from_numpy(c["x"]), CT.from_numpy(c["gy"]), CT(), CT()
        THNN.Threshold_updateOutput(x, ty, th, val, False)
        THNN.Threshold_updateGradInput(x, gy, tgx, th, val, False)
        y, gx = ty.numpy(), tgx.numpy()
    assert np.array_equal(y, c["y"]) and np.array_equal(gx, c["gx"])   # bit-exact: a select, no arithmetic


def test_batchnorm_relu_golden(backend):
    """The pair BatchNormalization (train) -> Threshold(0, 0): the oracle as the composition of its two functions, the
    library through its fused entry points (include/THCUNN_fused.h)."""
    c = case("bnrelu_4d")
    C = c["g"].shape[0]
    if backend.name == "oracle":
        rm, rv = np.zeros(C, np.float32), np.ones(C, np.float32)
        y, sm, ss = O.bn_updateOutput(c["x"], c["g"], c["b"], rm, rv, True, 0.1, 1e-5)
        a = O.threshold_updateOutput(y, 0.0, 0.0)
        gx, gw, gb = O.bn_backward(c["x"], O.threshold_updateGradInput(y, c["ga"], 0.0), c["g"], rm, rv, sm, ss, True, 1.0, 1e-5,
                                   np.zeros(C, np.float32), np.zeros(C, np.float32))
    else:
        CT, _, THNN = _hip()
        x, g, b, ga = (CT.from_numpy(c[k]) for k in ("x", "g", "b", "ga"))
        rm, rv = CT.from_numpy(np.zeros(C, np.float32)), CT.from_numpy(np.ones(C, np.float32))
        sm, ss, ta, tgx = CT.with_size(C), CT.with_size(C), CT(), CT.with_size(*c["x"].shape)
        tgw, tgb = CT.from_numpy(np.zeros(C, np.float32)), CT.from_numpy(np.zeros(C, np.float32))
        THNN.BatchNormalizationReLU_updateOutput(x, ta, g, b, rm, rv, sm, ss, True, 0.1, 1e-5)
        THNN.BatchNormalizationReLU_backward(x, ga, tgx, tgw, tgb, g, b, rm, rv, sm, ss, True, 1.0, 1e-5)
        a, gx, gw, gb = ta.numpy(), tgx.numpy(), tgw.numpy(), tgb.numpy()
    close(a, c["a"], 1e-5, 1e-4); close(gx, c["gx"], 1e-5, 1e-4); close(gw, c["gw"], 1e-3, 1e-3); close(gb, c["gb"], 1e-3, 1e-3)

"""The entry points under HIP graph capture: once the result and buffer tensors have their sizes, a call neither
allocates nor synchronises, so a caller may capture a sequence of calls on the state's stream and replay it.
The captured sequence is replayed three times, with the program's own eager calls and synchronisations between
the replays, and every replay has to give the eager results bit for bit. The depthwise weight gradient is
captured through its no-allocation variant (the one meant for such callers) and through the regular entry point
with the caller's scratch tensor already sized. BatchNormalization, which has no buffer argument, is captured on
both of its kernel families: 48 channels of 14 x 14 take the chunked two-pass kernels, whose chunk statistics
live in the state's per-stream scratch space (sized by the eager calls before the capture), 96 channels of
28 x 28 the kernels that keep a channel in registers.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_replays_of_a_captured_step_match_eager():
    import cunn_amd as T
    from cunn_amd.tensor import check, state
    CT, LT = T.CudaTensor, T.CudaLongTensor
    lib = T._lib.load()
    hip = C.CDLL("libamdhip64.so")
    rng = np.random.default_rng(5)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    N, Cd = 4, 32
    dw = dict(x=CT.from_numpy(f(N, Cd, 56, 56)), w=CT.from_numpy(f(1, Cd, 3, 3)), b=CT.from_numpy(f(1, Cd)), gy=CT.from_numpy(f(N, Cd, 28, 28)),
              y=CT(), gx=CT(), gw=CT.from_numpy(np.zeros((1, Cd, 3, 3), np.float32)), gb=CT.from_numpy(np.zeros((1, Cd), np.float32)),
              gw2=CT.from_numpy(np.zeros((1, Cd, 3, 3), np.float32)), gb2=CT.from_numpy(np.zeros((1, Cd), np.float32)), cols=CT(), ones=CT())
    Ci, Co = 64, 96
    cv = dict(x=CT.from_numpy(f(N, Ci, 28, 28)), w=CT.from_numpy(f(Co, Ci * 9) * 0.05), b=CT.from_numpy(f(Co)), gy=CT.from_numpy(f(N, Co, 28, 28)),
              y=CT(), gx=CT(), gw=CT.from_numpy(np.zeros((Co, Ci * 9), np.float32)), gb=CT.from_numpy(np.zeros(Co, np.float32)),
              cols=CT(), gcols=CT(), wcols=CT(), ones=CT())
    def make_bn(Cb, hw):
        z = lambda: CT.from_numpy(np.zeros(Cb, np.float32))
        return dict(x=CT.from_numpy(f(N, Cb, hw, hw)), gy=CT.from_numpy(f(N, Cb, hw, hw)), y=CT(), gx=CT.with_size(N, Cb, hw, hw),
                    g=CT.from_numpy(rng.random(Cb).astype(np.float32)), b=CT.from_numpy(f(Cb)), rm=z(),
                    rv=CT.from_numpy(np.ones(Cb, np.float32)), sm=CT.with_size(Cb), ss=CT.with_size(Cb), gw=z(), gb=z())

    bn, bn2 = make_bn(48, 14), make_bn(96, 28)
    mp = dict(x=CT.from_numpy(f(N, 16, 57, 57)), y=CT(), idx=LT(), gy=CT.from_numpy(f(N, 16, 29, 29)), gx=CT())
    h = lambda t: None if t is None else t.handle
    st = state()
    g, c = (3, 3, 2, 2, 1, 1), (3, 3, 1, 1, 1, 1)

    def step():
        lib.THNN_CudaSpatialDepthWiseConvolution_updateOutput(st, h(dw["x"]), h(dw["y"]), h(dw["w"]), h(dw["b"]), h(dw["cols"]), h(dw["ones"]), *g)
        lib.THNN_CudaSpatialDepthWiseConvolution_updateGradInput(st, h(dw["x"]), h(dw["gy"]), h(dw["gx"]), h(dw["w"]), h(dw["cols"]), h(dw["ones"]), *g)
        for k in ("gw", "gb", "gw2", "gb2"):
            lib.THCudaTensor_fill(st, h(dw[k]), 0.0)
        lib.THNN_CudaSpatialDepthWiseConvolution_accGradParameters_noAlloc(st, h(dw["x"]), h(dw["gy"]), h(dw["gw"]), h(dw["gb"]), *g, 1.0)
        lib.THNN_CudaSpatialDepthWiseConvolution_accGradParameters(st, h(dw["x"]), h(dw["gy"]), h(dw["gw2"]), h(dw["gb2"]), h(dw["cols"]), h(dw["ones"]), *g, 1.0)
        lib.THNN_CudaSpatialConvolutionMM_updateOutput(st, h(cv["x"]), h(cv["y"]), h(cv["w"]), h(cv["b"]), h(cv["cols"]), h(cv["ones"]), *c)
        lib.THNN_CudaSpatialConvolutionMM_updateGradInput(st, h(cv["x"]), h(cv["gy"]), h(cv["gx"]), h(cv["w"]), h(cv["gcols"]), h(cv["ones"]), *c)
        lib.THCudaTensor_fill(st, h(cv["gw"]), 0.0)
        lib.THCudaTensor_fill(st, h(cv["gb"]), 0.0)
        lib.THNN_CudaSpatialConvolutionMM_accGradParameters(st, h(cv["x"]), h(cv["gy"]), h(cv["gw"]), h(cv["gb"]), h(cv["wcols"]), h(cv["ones"]), *c, 1.0)
        for b_ in (bn, bn2):
            lib.THCudaTensor_fill(st, h(b_["rm"]), 0.0)
            lib.THCudaTensor_fill(st, h(b_["rv"]), 1.0)
            lib.THNN_CudaBatchNormalization_updateOutput(st, h(b_["x"]), h(b_["y"]), h(b_["g"]), h(b_["b"]), h(b_["rm"]), h(b_["rv"]), h(b_["sm"]), h(b_["ss"]), True, 0.1, 1e-5)
            lib.THCudaTensor_fill(st, h(b_["gw"]), 0.0)
            lib.THCudaTensor_fill(st, h(b_["gb"]), 0.0)
            lib.THNN_CudaBatchNormalization_backward(st, h(b_["x"]), h(b_["gy"]), h(b_["gx"]), h(b_["gw"]), h(b_["gb"]), h(b_["g"]), h(b_["rm"]), h(b_["rv"]), h(b_["sm"]), h(b_["ss"]), True, 1.0, 1e-5)
        lib.THNN_CudaSpatialMaxPooling_updateOutput(st, h(mp["x"]), h(mp["y"]), h(mp["idx"]), 3, 3, 2, 2, 1, 1, False)
        lib.THNN_CudaSpatialMaxPooling_updateGradInput(st, h(mp["x"]), h(mp["gy"]), h(mp["gx"]), h(mp["idx"]), 3, 3, 2, 2, 1, 1, False)

    outs = [dw["y"], dw["gx"], dw["gw"], dw["gb"], dw["gw2"], dw["gb2"], cv["y"], cv["gx"], cv["gw"], cv["gb"], bn["y"], bn["gx"], bn["gw"],
            bn["gb"], bn["rm"], bn["rv"], bn["sm"], bn["ss"], bn2["y"], bn2["gx"], bn2["gw"], bn2["gb"], bn2["sm"], bn2["ss"],
            mp["y"], mp["idx"], mp["gx"]]
    results = lambda: [t.numpy().copy() for t in outs]

    def scribble():
        """Eager work between replays: overwrite every result, so that a replay that did nothing would be seen."""
        for t in outs:
            if t is not mp["idx"]:
                lib.THCudaTensor_fill(st, h(t), -7.0)
        lib.THCState_synchronize(st)

    # a stream of the caller's own: the legacy default stream cannot be captured
    s = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(s)) == 0
    lib.THCState_setCurrentStream(st, s)
    try:
        step()                      # eager: sizes every result and scratch tensor
        step()
        lib.THCState_synchronize(st)
        check()
        expected = results()
        assert np.array_equal(expected[2], expected[4]) and np.array_equal(expected[3], expected[5])  # both depthwise weight-gradient entry points
        graph, graph_exec = C.c_void_p(), C.c_void_p()
        assert hip.hipStreamBeginCapture(s, 0) == 0
        step()
        assert hip.hipStreamEndCapture(s, C.byref(graph)) == 0
        check()
        assert hip.hipGraphInstantiate(C.byref(graph_exec), graph, None, None, C.c_size_t(0)) == 0
        for replay in range(3):
            scribble()
            assert hip.hipGraphLaunch(graph_exec, s) == 0
            lib.THCState_synchronize(st)
            for k, (got, want) in enumerate(zip(results(), expected)):
                assert np.array_equal(got, want), (replay, k)
            step()                  # eager calls between the replays
            lib.THCState_synchronize(st)
        assert hip.hipGraphExecDestroy(graph_exec) == 0 and hip.hipGraphDestroy(graph) == 0
    finally:
        lib.THCState_synchronize(st)
        lib.THCState_setCurrentStream(st, None)
        hip.hipStreamDestroy(s)
    check()

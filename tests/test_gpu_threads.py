"""Two host threads, each with its own THCState on its own HIP stream, drive different entry points at the same
time (ctypes releases the interpreter lock for the length of a call, and the kernels of the two streams share
the GPU). Every result has to equal, bit for bit, what the same calls give on the process-wide state alone: the
library keeps no state between calls except read-only caches, scratch lives in the caller's buffer tensors or
in stream-ordered temporaries, and no kernel uses atomics.
"""
import ctypes as C
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROUNDS = 8


def _workload(T, seed, shape_shift):
    """Tensors and calls of one thread: depthwise convolution (three passes, the weight gradient through the
    caller's scratch tensor), SpatialConvolutionMM (three passes: bordered copy, K-split partials and their
    fold in `columns`), BatchNormalization forward + backward, max pooling forward + backward."""
    CT, LT = T.CudaTensor, T.CudaLongTensor
    rng = np.random.default_rng(seed)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    N, C_, H = 4 + shape_shift, 32, 56
    dw = dict(x=CT.from_numpy(f(N, C_, H, H)), w=CT.from_numpy(f(1, C_, 3, 3)), b=CT.from_numpy(f(1, C_)),
              gy=CT.from_numpy(f(N, C_, 28, 28)), y=CT(), gx=CT(), gw=CT.from_numpy(np.zeros((1, C_, 3, 3), np.float32)),
              gb=CT.from_numpy(np.zeros((1, C_), np.float32)), cols=CT(), ones=CT())
    Ci, Co, P = 64, 64 + 32 * shape_shift, 28
    cv = dict(x=CT.from_numpy(f(N, Ci, P, P)), w=CT.from_numpy(f(Co, Ci * 9) * 0.05), b=CT.from_numpy(f(Co)),
              gy=CT.from_numpy(f(N, Co, P, P)), y=CT(), gx=CT(), gw=CT.from_numpy(np.zeros((Co, Ci * 9), np.float32)),
              gb=CT.from_numpy(np.zeros(Co, np.float32)), cols=CT(), ones=CT())
    Cb = 48
    z = lambda: CT.from_numpy(np.zeros(Cb, np.float32))
    bn = dict(x=CT.from_numpy(f(N, Cb, 14, 14)), gy=CT.from_numpy(f(N, Cb, 14, 14)), y=CT(), gx=CT.with_size(N, Cb, 14, 14),
              g=CT.from_numpy(rng.random(Cb).astype(np.float32)), b=CT.from_numpy(f(Cb)), rm=z(),
              rv=CT.from_numpy(np.ones(Cb, np.float32)), sm=CT.with_size(Cb), ss=CT.with_size(Cb), gw=z(), gb=z())
    mp = dict(x=CT.from_numpy(f(N, 16, 57, 57)), y=CT(), idx=LT(), gy=CT.from_numpy(f(N, 16, 29, 29)), gx=CT())
    h = lambda t: None if t is None else t.handle
    g = (3, 3, 2, 2, 1, 1)

    def calls(lib, st):
        lib.THNN_CudaSpatialDepthWiseConvolution_updateOutput(st, h(dw["x"]), h(dw["y"]), h(dw["w"]), h(dw["b"]), h(dw["cols"]), h(dw["ones"]), *g)
        lib.THNN_CudaSpatialDepthWiseConvolution_updateGradInput(st, h(dw["x"]), h(dw["gy"]), h(dw["gx"]), h(dw["w"]), h(dw["cols"]), h(dw["ones"]), *g)
        lib.THCudaTensor_fill(st, h(dw["gw"]), 0.0)
        lib.THCudaTensor_fill(st, h(dw["gb"]), 0.0)
        lib.THNN_CudaSpatialDepthWiseConvolution_accGradParameters(st, h(dw["x"]), h(dw["gy"]), h(dw["gw"]), h(dw["gb"]), h(dw["cols"]), h(dw["ones"]), *g, 1.0)
        c = (3, 3, 1, 1, 1, 1)
        lib.THNN_CudaSpatialConvolutionMM_updateOutput(st, h(cv["x"]), h(cv["y"]), h(cv["w"]), h(cv["b"]), h(cv["cols"]), h(cv["ones"]), *c)
        lib.THNN_CudaSpatialConvolutionMM_updateGradInput(st, h(cv["x"]), h(cv["gy"]), h(cv["gx"]), h(cv["w"]), h(cv["cols"]), h(cv["ones"]), *c)
        lib.THCudaTensor_fill(st, h(cv["gw"]), 0.0)
        lib.THCudaTensor_fill(st, h(cv["gb"]), 0.0)
        lib.THNN_CudaSpatialConvolutionMM_accGradParameters(st, h(cv["x"]), h(cv["gy"]), h(cv["gw"]), h(cv["gb"]), h(cv["cols"]), h(cv["ones"]), *c, 1.0)
        lib.THCudaTensor_fill(st, h(bn["rm"]), 0.0)
        lib.THCudaTensor_fill(st, h(bn["rv"]), 1.0)
        lib.THNN_CudaBatchNormalization_updateOutput(st, h(bn["x"]), h(bn["y"]), h(bn["g"]), h(bn["b"]), h(bn["rm"]), h(bn["rv"]), h(bn["sm"]), h(bn["ss"]), True, 0.1, 1e-5)
        lib.THCudaTensor_fill(st, h(bn["gw"]), 0.0)
        lib.THCudaTensor_fill(st, h(bn["gb"]), 0.0)
        lib.THNN_CudaBatchNormalization_backward(st, h(bn["x"]), h(bn["gy"]), h(bn["gx"]), h(bn["gw"]), h(bn["gb"]), h(bn["g"]), h(bn["rm"]), h(bn["rv"]), h(bn["sm"]), h(bn["ss"]), True, 1.0, 1e-5)
        lib.THNN_CudaSpatialMaxPooling_updateOutput(st, h(mp["x"]), h(mp["y"]), h(mp["idx"]), 3, 3, 2, 2, 1, 1, False)
        lib.THNN_CudaSpatialMaxPooling_updateGradInput(st, h(mp["x"]), h(mp["gy"]), h(mp["gx"]), h(mp["idx"]), 3, 3, 2, 2, 1, 1, False)

    def results():
        outs = [dw["y"], dw["gx"], dw["gw"], dw["gb"], cv["y"], cv["gx"], cv["gw"], cv["gb"], bn["y"], bn["gx"], bn["gw"], bn["gb"],
                bn["rm"], bn["rv"], bn["sm"], bn["ss"], mp["y"], mp["idx"], mp["gx"]]
        return [t.numpy().copy() for t in outs]

    return calls, results


def test_two_states_two_streams_two_threads():
    import cunn_amd as T
    from cunn_amd.tensor import check, state
    lib = T._lib.load()
    hip = C.CDLL("libamdhip64.so")
    work = [_workload(T, 100 + i, i) for i in range(2)]
    # what each workload gives alone, on the process-wide state
    expected = []
    for calls, results in work:
        calls(lib, state())
        lib.THCState_synchronize(state())
        check()
        expected.append(results())
    streams, states = [], []
    for _ in work:
        s = C.c_void_p()
        assert hip.hipStreamCreate(C.byref(s)) == 0   # default priority
        st = lib.THCState_alloc()
        lib.THCState_setCurrentStream(st, s)
        streams.append(s), states.append(st)
    errors = []

    def run(i):
        try:
            for _ in range(ROUNDS):
                work[i][0](lib, states[i])
            lib.THCState_synchronize(states[i])
        except Exception as e:  # noqa: BLE001
            errors.append(e)

    threads = [threading.Thread(target=run, args=(i,)) for i in range(len(work))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    check()
    assert not errors, errors
    for i, (_, results) in enumerate(work):
        for k, (got, want) in enumerate(zip(results(), expected[i])):
            assert got.shape == want.shape and np.array_equal(got, want), (i, k)
    for st, s in zip(states, streams):
        lib.THCState_free(st)
        assert hip.hipStreamDestroy(s) == 0

"""updateGradInput of convolutions with one to four input planes (and the forward pass of transposed convolutions
with one to four output planes) runs on a kernel of its own, built on 4x4 matrix instructions, instead of gradient
columns + col2im (lib/THCUNN/generic/SpatialConvolutionMM.cu:272-308, lib/THCUNN/im2col.h:63-102).
Every compiled kernel size, the run-time tap loops on the same geometries, ragged blocks, every phase count,
against the oracle through the C ABI."""
import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402


def out_size(i, k, d, p):
    return (i + 2 * p - k) // d + 1


# N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH
COMPILED = [
    (2, 3, 16, 40, 40, 7, 7, 2, 2, 3, 3),      # 7x7 stride 2 (first layer of ResNet)
    (3, 3, 10, 37, 45, 7, 7, 2, 2, 3, 3),      # odd extents: the phases have different sizes; 10 planes: a chunk of 2
    (2, 3, 8, 34, 34, 3, 3, 2, 2, 1, 1),       # 3x3 stride 2 pad 1
    (2, 3, 8, 35, 35, 3, 3, 2, 2, 0, 0),       # 3x3 stride 2 unpadded
    (2, 3, 12, 40, 24, 3, 3, 1, 1, 1, 1),      # 3x3
    (2, 1, 6, 33, 19, 3, 3, 1, 1, 1, 1),       # one input plane
    (2, 4, 9, 20, 20, 5, 5, 1, 1, 2, 2),       # 5x5, four planes
    (2, 2, 7, 36, 36, 4, 4, 2, 2, 1, 1),       # 4x4 stride 2
    (2, 3, 6, 67, 67, 11, 11, 4, 4, 2, 2),     # 11x11 stride 4 (AlexNet)
    (1, 3, 5, 9, 7, 7, 7, 2, 2, 3, 3),         # smaller than one block
    (2, 3, 64, 96, 96, 7, 7, 2, 2, 3, 3),      # several blocks per image in both directions, 16 chunks
]
RUNTIME = [
    (2, 3, 8, 30, 30, 5, 5, 2, 2, 2, 2),       # 5x5 stride 2
    (2, 3, 8, 30, 26, 3, 5, 1, 1, 2, 1),       # rectangular kernel, different paddings (kW=3, kH=5)
    (2, 2, 8, 31, 31, 6, 6, 3, 3, 2, 2),       # stride 3: nine phases
    (2, 3, 8, 41, 41, 8, 8, 4, 4, 2, 2),       # stride 4 with another kernel size
    (2, 3, 8, 25, 25, 1, 1, 2, 2, 0, 0),       # 1x1 stride 2: three of four phases receive nothing
    (2, 4, 8, 22, 22, 2, 2, 2, 2, 0, 0),       # window = stride
    (2, 3, 8, 20, 20, 3, 3, 3, 3, 0, 0),
    (2, 3, 6, 28, 28, 9, 9, 1, 1, 4, 4),       # 9x9: the widest halo the parked patch takes
    (2, 3, 8, 33, 33, 3, 3, 2, 2, 2, 2),       # padding beyond k/2
]


def _grad_input(case, seed, modes):
    N, Ci, Co, H, W, kW, kH, dW, dH, pW, pH = case
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(seed)
    oH, oW = out_size(H, kH, dH, pH), out_size(W, kW, dW, pW)
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci * kH * kW)) * np.sqrt(2.0 / (Ci * kH * kW))).astype(np.float32)
    gy = rng.standard_normal((N, Co, oH, oW)).astype(np.float32)
    g = (kW, kH, dW, dH, pW, pH)
    ref = O.convmm_updateGradInput(x.shape, gy, w, *g)
    tx, tw, tgy = CT.from_numpy(x), CT.from_numpy(w), CT.from_numpy(gy)
    got = {}
    for mode in modes:
        cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", mode)
        try:
            gx = CT()
            THNN.SpatialConvolutionMM_updateGradInput(tx, tgy, gx, tw, CT(), CT(), *g)
            got[mode] = gx.numpy()
        finally:
            cunn_amd.set_switch("THCUNN_CONV_GRADINPUT", None)
        assert got[mode].shape == ref.shape
        np.testing.assert_allclose(got[mode], ref, rtol=1e-5, atol=1e-4, err_msg=f"route {mode}")
    return got


@pytest.mark.parametrize("case", COMPILED)
def test_compiled_kernel_sizes(case):
    """Default route (taps resolved at compile time), the run-time tap loops and the gradient-column route agree with
    the oracle; the two variants of the kernel add the same terms in the same order."""
    print("case", case, flush=True)
    got = _grad_input(case, 80, [None, "planes", "columns"])
    assert np.array_equal(got[None], got["planes"])


@pytest.mark.parametrize("case", RUNTIME)
def test_runtime_kernel_sizes(case):
    print("case", case, flush=True)
    _grad_input(case, 81, [None, "columns"])


def test_seeded_geometries():
    """Random kernel sizes, strides, paddings and extents (the ranges of the reference's SpatialConvolutionMM tests,
    test.lua, with 1..4 input planes)."""
    rng = np.random.default_rng(82)
    for it in range(40):
        s = int(rng.integers(1, 5))
        kW, kH = int(rng.integers(1, 8)), int(rng.integers(1, 8))
        pW, pH = int(rng.integers(0, kW // 2 + 1)), int(rng.integers(0, kH // 2 + 1))
        oW, oH = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        W, H = (oW - 1) * s + kW - 2 * pW + int(rng.integers(0, s)), (oH - 1) * s + kH - 2 * pH + int(rng.integers(0, s))
        if W < 1 or H < 1:
            continue
        case = (int(rng.integers(1, 4)), int(rng.integers(1, 5)), int(rng.integers(1, 12)), H, W, kW, kH, s, s, pW, pH)
        print("draw", it, case, flush=True)
        _grad_input(case, 1000 + it, [None])


# the forward pass of a transposed convolution is the same pass, with the bias added by the kernel:
# N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, adjW, adjH
FULL = [
    (2, 16, 3, 16, 16, 4, 4, 2, 2, 1, 1, 0, 0),   # the last layer of a generator: 16 -> 3 planes, 4x4 stride 2
    (2, 8, 1, 9, 11, 3, 3, 2, 2, 1, 1, 1, 1),     # output padding: rows that no window reaches hold the bias
    (2, 6, 4, 10, 10, 5, 5, 1, 1, 2, 2, 0, 0),
    (1, 5, 2, 7, 7, 6, 6, 3, 3, 1, 1, 2, 2),
]


@pytest.mark.parametrize("case", FULL)
@pytest.mark.parametrize("bias", [True, False])
def test_transposed_convolution_forward(case, bias):
    print("case", case, "bias", bias, flush=True)
    N, Ci, Co, H, W, kW, kH, dW, dH, pW, pH, aW, aH = case
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(83)
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Ci, Co, kH, kW)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32) if bias else None
    ref = O.fullconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH, 1, 1, aW, aH)
    out = CT()
    THNN.SpatialFullConvolution_updateOutput(CT.from_numpy(x), out, CT.from_numpy(w), CT.from_numpy(b) if bias else None,
                                             CT(), CT(), kW, kH, dW, dH, pW, pH, aW, aH)
    y = out.numpy()
    assert y.shape == ref.shape
    np.testing.assert_allclose(y, ref, rtol=1e-5, atol=1e-4)

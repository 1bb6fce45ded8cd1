"""Pins the CPU oracle (oracle/thnn_oracle.c) before it is trusted as a checker.

Three independent anchors per function:
  * closed-form brute force in float64 (tests/bruteforce.py) on tiny shapes;
  * PyTorch-CPU library routines + autograd on mid-size shapes;
  * the reference's own known answers / identities:
      - test.lua:2597-2616  SpatialAveragePooling 1x1 input 3, k2 s1 p1 -> 3 and 3/4
      - test.lua:6602-6661  depthwise == concat of per-channel SpatialConvolution
      - test.lua:2083-2085  indices equal the CPU indices (first maximum, 1-based)
and mathematical invariants (adjointness of im2col/col2im and of the conv
gradients, BN gradient orthogonality, max-pool index round trip).
"""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import bruteforce as bf
from oracle import oracle as O

RTOL, ATOL = 1e-5, 1e-4


def close(a, b, rtol=RTOL, atol=ATOL):
    np.testing.assert_allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), rtol=rtol, atol=atol)


# ------------------------------------------------------------ im2col/col2im --
@pytest.mark.parametrize("k,d,p,dil", [((3, 3), (1, 1), (1, 1), (1, 1)), ((2, 4), (2, 1), (0, 1), (1, 1)),
                                       ((3, 2), (2, 3), (1, 0), (2, 1)), ((5, 3), (1, 2), (2, 1), (1, 2))])
def test_im2col_definition_and_adjoint(k, d, p, dil):
    rng = np.random.default_rng(0)
    kH, kW = k; dH, dW = d; pH, pW = p; dlH, dlW = dil
    C, H, W = 3, 9, 11
    im = rng.standard_normal((C, H, W)).astype(np.float32)
    col = O.im2col(im, kW, kH, dW, dH, pW, pH, dlW, dlH)
    oH = O.conv_out_size(H, kH, dH, pH, dlH); oW = O.conv_out_size(W, kW, dW, pW, dlW)
    ref = np.zeros((C, kH, kW, oH, oW), np.float32)
    for c, i, j, oh, ow in itertools.product(range(C), range(kH), range(kW), range(oH), range(oW)):
        h, w = oh * dH - pH + i * dlH, ow * dW - pW + j * dlW
        if 0 <= h < H and 0 <= w < W:
            ref[c, i, j, oh, ow] = im[c, h, w]
    assert np.array_equal(col, ref.reshape(C * kH * kW, oH * oW))
    # col2im is the exact transpose of im2col: <im2col(a), b> == <a, col2im(b)>
    b = rng.standard_normal(col.shape).astype(np.float32)
    back = O.col2im(b, C, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH)
    close(np.vdot(col.astype(np.float64), b), np.vdot(im.astype(np.float64), back), 1e-5, 1e-4)


# ------------------------------------------------------------------ depthwise --
DW_CASES = [  # N, C, M, H, W, kW, kH, dW, dH, padW, padH
    (2, 3, 1, 7, 8, 3, 3, 1, 1, 1, 1),
    (1, 2, 4, 6, 5, 3, 2, 2, 1, 0, 1),
    (2, 2, 2, 9, 9, 3, 3, 2, 2, 1, 1),
    (1, 1, 3, 5, 7, 1, 4, 1, 3, 0, 2),
]


@pytest.mark.parametrize("case", DW_CASES)
@pytest.mark.parametrize("with_bias", [True, False])
def test_dwconv_bruteforce(case, with_bias):
    N, C, M, H, W, kW, kH, dW, dH, pW, pH = case
    rng = np.random.default_rng(1)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    w = rng.standard_normal((M, C, kH, kW)).astype(np.float32)
    b = rng.standard_normal((M, C)).astype(np.float32) if with_bias else None
    y = O.dwconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH)
    close(y, bf.dw_forward(x, w, b, dW, dH, pW, pH))
    gy = rng.standard_normal(y.shape).astype(np.float32)
    close(O.dwconv_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH),
          bf.dw_grad_input(x.shape, gy, w, dW, dH, pW, pH))
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    gb0 = rng.standard_normal((M, C)).astype(np.float32)
    gw, gb = O.dwconv_accGradParameters(x, gy, gw0.copy(), gb0.copy(), kW, kH, dW, dH, pW, pH, scale=0.5)
    rgw, rgb = bf.dw_grad_params(x, gy, M, kW, kH, dW, dH, pW, pH)
    close(gw, gw0 + 0.5 * rgw, 1e-4, 1e-4)  # accumulates into the existing values
    close(gb, gb0 + 0.5 * rgb, 1e-4, 1e-4)


def test_dwconv_equals_per_channel_convolution():
    """The identity the reference's only depthwise test asserts (test.lua:6602-6661):
    n=3 planes, multiplier 4, 28x28, k3 s1 p1, batch 3; the comparison model runs one
    SpatialConvolution(1 -> m) per input channel with weight:narrow(2, c, 1) and
    bias:select(2, c), concatenated along the channel axis. eps 1e-5."""
    rng = np.random.default_rng(2)
    n, s, b, m, k, p, st = 3, 28, 3, 4, 3, 1, 1
    X = rng.random((b, n, s, s), dtype=np.float32)
    weight = rng.random((m, n, k, k), dtype=np.float32)
    bias = rng.random((m, n), dtype=np.float32)
    Y = O.dwconv_updateOutput(X, weight, bias, k, k, st, st, p, p)
    parts = []
    for c in range(n):
        wc = torch.from_numpy(weight[:, c:c + 1].copy())      # (m, 1, k, k)
        bc = torch.from_numpy(bias[:, c].copy())               # (m,)
        parts.append(F.conv2d(torch.from_numpy(X[:, c:c + 1].copy()), wc, bc, stride=st, padding=p))
    Y_util = torch.cat(parts, dim=1).numpy()
    assert np.all(np.abs(Y_util - Y) < 1e-5)
    # the same identity through the oracle's own dense path
    for c in range(n):
        yc = O.convmm_updateOutput(X[:, c:c + 1], weight[:, c].reshape(m, k * k), bias[:, c], k, k, st, st, p, p)
        assert np.all(np.abs(yc - Y[:, c * m:(c + 1) * m]) < 1e-5)


@pytest.mark.parametrize("case", [(4, 16, 1, 28, 28, 3, 3, 2, 2, 1, 1), (2, 8, 2, 19, 23, 5, 3, 1, 2, 2, 1)])
def test_dwconv_vs_torch_grouped_conv(case):
    N, C, M, H, W, kW, kH, dW, dH, pW, pH = case
    rng = np.random.default_rng(3)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    w = rng.standard_normal((M, C, kH, kW)).astype(np.float32)
    b = rng.standard_normal((M, C)).astype(np.float32)
    # reference weight[j][c] <-> torch grouped weight[c*M + j][0]; bias[j][c] <-> bias[c*M + j]
    tw = torch.from_numpy(w.transpose(1, 0, 2, 3).reshape(C * M, 1, kH, kW).copy()).double().requires_grad_()
    tb = torch.from_numpy(b.T.reshape(C * M).copy()).double().requires_grad_()
    tx = torch.from_numpy(x).double().requires_grad_()
    ty = F.conv2d(tx, tw, tb, stride=(dH, dW), padding=(pH, pW), groups=C)
    y = O.dwconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH)
    close(y, ty.detach().numpy())
    gy = rng.standard_normal(y.shape).astype(np.float32)
    ty.backward(torch.from_numpy(gy).double())
    close(O.dwconv_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH), tx.grad.numpy())
    gw, gb = O.dwconv_accGradParameters(x, gy, np.zeros_like(w), np.zeros_like(b), kW, kH, dW, dH, pW, pH, 1.0)
    close(gw, tw.grad.numpy().reshape(C, M, kH, kW).transpose(1, 0, 2, 3), 1e-3, 1e-4)
    close(gb, tb.grad.numpy().reshape(C, M).T, 1e-3, 1e-4)


# --------------------------------------------------------------------- ConvMM --
@pytest.mark.parametrize("case", [(2, 3, 4, 7, 6, 3, 3, 1, 1, 1, 1), (1, 2, 8, 9, 10, 4, 3, 2, 3, 1, 0),
                                  (3, 5, 2, 8, 8, 2, 5, 1, 2, 0, 1)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_convmm_bruteforce_and_adjoint(case, with_bias):
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH = case
    rng = np.random.default_rng(4)
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = rng.standard_normal((Cout, Cin * kH * kW)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32) if with_bias else None
    y = O.convmm_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH)
    close(y, bf.conv_forward(x, w.reshape(Cout, Cin, kH, kW), b, dW, dH, pW, pH))
    gy = rng.standard_normal(y.shape).astype(np.float32)
    gx = O.convmm_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH)
    gw, gb = O.convmm_accGradParameters(x, gy, np.zeros_like(w), np.zeros(Cout, np.float32), kW, kH, dW, dH, pW, pH)
    y0 = O.convmm_updateOutput(x, w, None, kW, kH, dW, dH, pW, pH).astype(np.float64)
    # <conv(x), gy> = <x, gradInput(gy)> = <W, gradW>
    lhs = np.vdot(y0, gy)
    close(lhs, np.vdot(x.astype(np.float64), gx), 1e-4, 1e-3)
    close(lhs, np.vdot(w.astype(np.float64), gw), 1e-4, 1e-3)
    close(gb, gy.astype(np.float64).sum(axis=(0, 2, 3)), 1e-4, 1e-4)


def test_convmm_vs_torch_autograd():
    rng = np.random.default_rng(5)
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH = 4, 6, 16, 13, 17, 3, 5, 2, 1, 1, 2
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kH, kW)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    tx = torch.from_numpy(x).double().requires_grad_()
    tw = torch.from_numpy(w).double().requires_grad_()
    tb = torch.from_numpy(b).double().requires_grad_()
    ty = F.conv2d(tx, tw, tb, stride=(dH, dW), padding=(pH, pW))
    y = O.convmm_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH)
    close(y, ty.detach().numpy())
    gy = rng.standard_normal(y.shape).astype(np.float32)
    ty.backward(torch.from_numpy(gy).double())
    close(O.convmm_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH), tx.grad.numpy())
    gw0 = rng.standard_normal((Cout, Cin * kH * kW)).astype(np.float32)
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    gw, gb = O.convmm_accGradParameters(x, gy, gw0.copy(), gb0.copy(), kW, kH, dW, dH, pW, pH, scale=2.0)
    close(gw, gw0 + 2.0 * tw.grad.numpy().reshape(Cout, -1), 1e-3, 1e-3)
    close(gb, gb0 + 2.0 * tb.grad.numpy(), 1e-3, 1e-3)


# ------------------------------------------------ dilated / transposed conv --
DIL_CASES = [
    # N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH
    (2, 3, 4, 13, 15, 3, 3, 1, 1, 2, 2, 2, 2),
    (2, 2, 5, 17, 14, 3, 2, 2, 1, 1, 0, 3, 2),
    (1, 4, 3, 11, 11, 2, 3, 1, 2, 0, 3, 1, 3),
]


@pytest.mark.parametrize("case", DIL_CASES)
def test_dilconv_vs_torch_autograd_and_adjoint(case):
    """SpatialDilatedConvolution restated: float64 torch conv2d(dilation=) + autograd fixes the
    values; dilation 1 reduces to SpatialConvolutionMM; <conv(x),gy> = <x,gradInput> = <W,gradW>."""
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH = case
    rng = np.random.default_rng(70)
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, kH, kW)) * 0.3).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    tx = torch.from_numpy(x).double().requires_grad_()
    tw = torch.from_numpy(w).double().requires_grad_()
    tb = torch.from_numpy(b).double().requires_grad_()
    ty = F.conv2d(tx, tw, tb, stride=(dH, dW), padding=(pH, pW), dilation=(dlH, dlW))
    y = O.dilconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH, dlW, dlH)
    close(y, ty.detach().numpy())
    gy = rng.standard_normal(y.shape).astype(np.float32)
    ty.backward(torch.from_numpy(gy).double())
    gx = O.dilconv_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH, dlW, dlH)
    close(gx, tx.grad.numpy())
    gw0 = rng.standard_normal((Cout, Cin * kH * kW)).astype(np.float32)
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    gw, gb = O.dilconv_accGradParameters(x, gy, gw0.copy(), gb0.copy(), kW, kH, dW, dH, pW, pH, dlW, dlH, scale=0.5)
    close(gw, gw0 + 0.5 * tw.grad.numpy().reshape(Cout, -1), 1e-3, 1e-3)
    close(gb, gb0 + 0.5 * tb.grad.numpy(), 1e-3, 1e-3)
    y1 = O.dilconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH, 1, 1)
    assert np.array_equal(y1, O.convmm_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH))


FULL_CASES = [
    # N, Cin, Cout, H, W, kW, kH, dW, dH, padW, padH, dilW, dilH, adjW, adjH
    (2, 3, 4, 7, 9, 3, 3, 2, 2, 1, 1, 1, 1, 1, 1),
    (2, 4, 2, 6, 5, 4, 3, 1, 1, 0, 1, 1, 1, 0, 0),
    (1, 2, 3, 5, 6, 3, 2, 3, 2, 1, 0, 2, 2, 2, 1),
    (2, 2, 2, 4, 4, 2, 2, 2, 2, 0, 0, 1, 1, 0, 0),
]


@pytest.mark.parametrize("case", FULL_CASES)
def test_fullconv_vs_torch_and_transpose_identity(case):
    """SpatialFull(Dilated)Convolution restated: float64 conv_transpose2d + autograd fixes the
    values; the forward pass is the adjoint of the ordinary convolution with the same weight
    read as (Cout_conv = Cin, Cin_conv = Cout): <full(x), z> = <x, conv(z)>."""
    N, Cin, Cout, H, W, kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH = case
    rng = np.random.default_rng(71)
    x = rng.standard_normal((N, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cin, Cout, kH, kW)) * 0.3).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    tx = torch.from_numpy(x).double().requires_grad_()
    tw = torch.from_numpy(w).double().requires_grad_()
    tb = torch.from_numpy(b).double().requires_grad_()
    ty = F.conv_transpose2d(tx, tw, tb, stride=(dH, dW), padding=(pH, pW), output_padding=(aH, aW),
                            dilation=(dlH, dlW))
    y = O.fullconv_updateOutput(x, w, b, kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH)
    assert y.shape == tuple(ty.shape)
    close(y, ty.detach().numpy())
    gy = rng.standard_normal(y.shape).astype(np.float32)
    ty.backward(torch.from_numpy(gy).double())
    gx = O.fullconv_updateGradInput(x.shape, gy, w, kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH)
    close(gx, tx.grad.numpy())
    gw0 = rng.standard_normal(w.shape).astype(np.float32)
    gb0 = rng.standard_normal(Cout).astype(np.float32)
    gw, gb = O.fullconv_accGradParameters(x, gy, gw0.copy(), gb0.copy(), kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH,
                                          scale=1.5)
    close(gw, gw0 + 1.5 * tw.grad.numpy(), 1e-3, 1e-3)
    close(gb, gb0 + 1.5 * tb.grad.numpy(), 1e-3, 1e-3)
    # adjoint of the ordinary (dilated) convolution over the output-sized image
    z = rng.standard_normal(y.shape).astype(np.float32)
    cz = O.dilconv_updateOutput(z, w.reshape(Cin, Cout * kH * kW), None, kW, kH, dW, dH, pW, pH, dlW, dlH)
    y0 = O.fullconv_updateOutput(x, w, None, kW, kH, dW, dH, pW, pH, dlW, dlH, aW, aH)
    close(np.vdot(y0.astype(np.float64), z), np.vdot(x.astype(np.float64), cz[:, :, :H, :W]), 1e-4, 1e-3)


# ------------------------------------------------------------------------- BN --
@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("shape", [(4, 3, 5, 7), (2, 5, 1, 1), (8, 2, 6)])
def test_bn_train_textbook_and_invariants(shape, affine):
    rng = np.random.default_rng(6)
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    Cc = shape[1]
    g = rng.random(Cc).astype(np.float32) if affine else None
    b = rng.standard_normal(Cc).astype(np.float32) if affine else None
    rm = rng.standard_normal(Cc).astype(np.float32); rv = (rng.random(Cc) + 0.5).astype(np.float32)
    rm0, rv0 = rm.copy(), rv.copy()
    eps, mom = 1e-5, 0.1
    y, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, mom, eps)
    ry, mean, inv, var_u = bf.bn_forward(x, g, b, eps)
    close(y, ry)
    close(sm, mean, 1e-5, 1e-6)
    close(ss, inv, 1e-5, 1e-6)                       # saveStd holds 1/sigma
    close(rm, (1 - mom) * rm0 + mom * mean, 1e-5, 1e-6)
    close(rv, (1 - mom) * rv0 + mom * var_u, 1e-5, 1e-6)  # unbiased (n-1) variance
    gy = rng.standard_normal(shape).astype(np.float32)
    gw0 = rng.standard_normal(Cc).astype(np.float32); gb0 = rng.standard_normal(Cc).astype(np.float32)
    gi, gw, gb = O.bn_backward(x, gy, g, rm, rv, sm, ss, True, 0.7, eps, gw0.copy(), gb0.copy())
    rgx, rgw, rgb = bf.bn_backward(x, gy, g, mean, inv)
    close(gi, rgx, 1e-4, 1e-4)
    close(gw, gw0 + 0.7 * rgw, 1e-4, 1e-4)
    close(gb, gb0 + 0.7 * rgb, 1e-4, 1e-4)
    # train-mode gradient is orthogonal to 1 and to (x - mean) per channel
    gir = gi.reshape(shape[0], Cc, -1).astype(np.float64)
    xc = x.reshape(shape[0], Cc, -1) - mean[None, :, None]
    assert np.all(np.abs(gir.sum(axis=(0, 2))) < 1e-3)
    assert np.all(np.abs((gir * xc).sum(axis=(0, 2))) < 1e-2)


def test_bn_vs_torch_train_and_eval():
    rng = np.random.default_rng(7)
    shape = (6, 4, 9, 5)
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    g = rng.random(4).astype(np.float32); b = rng.standard_normal(4).astype(np.float32)
    rm = np.zeros(4, np.float32); rv = np.ones(4, np.float32)
    trm, trv = torch.zeros(4, dtype=torch.float64), torch.ones(4, dtype=torch.float64)
    tx = torch.from_numpy(x).double().requires_grad_()
    tg = torch.from_numpy(g).double().requires_grad_(); tb = torch.from_numpy(b).double().requires_grad_()
    ty = F.batch_norm(tx, trm, trv, tg, tb, True, 0.1, 1e-5)
    y, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, 0.1, 1e-5)
    close(y, ty.detach().numpy()); close(rm, trm.numpy(), 1e-5, 1e-6); close(rv, trv.numpy(), 1e-5, 1e-6)
    gy = rng.standard_normal(shape).astype(np.float32)
    ty.backward(torch.from_numpy(gy).double())
    gi, gw, gb = O.bn_backward(x, gy, g, rm, rv, sm, ss, True, 1.0, 1e-5, np.zeros(4, np.float32), np.zeros(4, np.float32))
    close(gi, tx.grad.numpy(), 1e-4, 1e-4); close(gw, tg.grad.numpy(), 1e-4, 1e-4); close(gb, tb.grad.numpy(), 1e-4, 1e-4)
    # evaluation mode: running statistics, gradInput = gy * gamma / sqrt(runVar + eps)
    ye, _, _ = O.bn_updateOutput(x, g, b, rm, rv, False, 0.1, 1e-5)
    close(ye, F.batch_norm(torch.from_numpy(x).double(), trm, trv, tg.detach(), tb.detach(), False, 0.1, 1e-5).numpy())
    gie, _, _ = O.bn_backward(x, gy, g, rm, rv, sm, ss, False, 1.0, 1e-5)
    close(gie, gy * (g / np.sqrt(rv.astype(np.float64) + 1e-5))[None, :, None, None])
    # split call order (updateGradInput then accGradParameters) == fused backward (test.lua:989-1003)
    gi2, _, _ = O.bn_backward(x, gy, g, rm, rv, sm, ss, True, 1.0, 1e-5)
    _, gw2, gb2 = O.bn_backward(x, gy, g, rm, rv, sm, ss, True, 1.0, 1e-5, np.zeros(4, np.float32), np.zeros(4, np.float32), want_gradInput=False)
    assert np.array_equal(gi, gi2) and np.array_equal(gw, gw2) and np.array_equal(gb, gb2)


def test_bn_eval_mode_parameter_gradients():
    """Evaluation mode takes mean and 1/sigma from the running statistics for the parameter gradients too
    (lib/THCUNN/BatchNormalization.cu:237-240, 272-282): gradWeight += scale * sum(gy * (x - runningMean)) /
    sqrt(runningVar + eps), gradBias += scale * sum(gy), on top of what the tensors held. Checked against those
    closed forms in float64 and against autograd through F.batch_norm(training=False), with running statistics
    that differ from the batch's and from (0, 1), a scale that is not 1 and accumulators that are not 0."""
    rng = np.random.default_rng(11)
    shape, C, eps, scale = (5, 3, 6, 7), 3, 1e-3, 0.75
    x = (rng.standard_normal(shape) * 1.5 - 0.3).astype(np.float32)
    gy = rng.standard_normal(shape).astype(np.float32)
    g = (rng.random(C) + 0.5).astype(np.float32)
    rm = rng.standard_normal(C).astype(np.float32)
    rv = (rng.random(C) * 2 + 0.25).astype(np.float32)
    gw0, gb0 = rng.standard_normal(C).astype(np.float32), rng.standard_normal(C).astype(np.float32)
    # saveMean / saveStd of some training step: must not enter the evaluation-mode formulas
    sm, ss = np.full(C, 123.0, np.float32), np.full(C, 456.0, np.float32)
    gi, gw, gb = O.bn_backward(x, gy, g, rm, rv, sm, ss, False, scale, eps, gw0.copy(), gb0.copy())
    x64, gy64 = x.astype(np.float64), gy.astype(np.float64)
    inv = 1.0 / np.sqrt(rv.astype(np.float64) + eps)
    want_gw = gw0 + scale * (gy64 * (x64 - rm[None, :, None, None])).sum(axis=(0, 2, 3)) * inv
    want_gb = gb0 + scale * gy64.sum(axis=(0, 2, 3))
    close(gw, want_gw, 1e-5, 1e-5); close(gb, want_gb, 1e-5, 1e-5)
    close(gi, gy64 * (g * inv)[None, :, None, None], 1e-5, 1e-6)
    tx = torch.from_numpy(x).double().requires_grad_()
    tg, tb = torch.from_numpy(g).double().requires_grad_(), torch.zeros(C, dtype=torch.float64, requires_grad=True)
    F.batch_norm(tx, torch.from_numpy(rm).double(), torch.from_numpy(rv).double(), tg, tb, False, 0.1, eps).backward(
        torch.from_numpy(gy).double())
    close(gw, gw0 + scale * tg.grad.numpy(), 1e-5, 1e-5); close(gb, gb0 + scale * tb.grad.numpy(), 1e-5, 1e-5)
    close(gi, tx.grad.numpy(), 1e-5, 1e-6)


def test_bn_zero_variance_zero_eps():
    """invStd = 0 when varN == 0 and eps == 0 (lib/THCUNN/BatchNormalization.cu:188-191)."""
    x = np.full((2, 1, 3), 4.0, np.float32)
    y, sm, ss = O.bn_updateOutput(x, None, None, np.zeros(1, np.float32), np.ones(1, np.float32), True, 0.1, 0.0)
    assert ss[0] == 0 and sm[0] == 4 and np.all(y == 0)


# -------------------------------------------------------------------- pooling --
def test_pool_out_size_rule_exhaustive():
    for n, k, d, ceil_mode in itertools.product(range(1, 20), range(1, 6), range(1, 5), (0, 1)):
        for p in range(0, k // 2 + 1):
            for dil in (1, 2):
                if n + 2 * p < dil * (k - 1) + 1:
                    continue
                for anyp in ({True} if p else {False, True}):
                    assert O.pool_out_size(n, k, d, p, dil, ceil_mode, anyp) == bf.pool_out(n, k, d, p, dil, ceil_mode, anyp)


def test_avgpool_reference_known_answer():
    """test.lua:2597-2616: SpatialAveragePooling(2,2,1,1,1,1) on a 1x1x1x1 input holding 3."""
    x = np.full((1, 1, 1, 1), 3.0, np.float32)
    noinc = O.avgpool_updateOutput(x, 2, 2, 1, 1, 1, 1, False, False)
    inc = O.avgpool_updateOutput(x, 2, 2, 1, 1, 1, 1, False, True)
    assert noinc[0, 0, 0, 0] == 3.0
    assert inc[0, 0, 0, 0] == 3.0 / 4
    assert noinc[0, 0, 0, 0] != inc[0, 0, 0, 0]


POOL_CASES = [  # H, W, kW, kH, dW, dH, padW, padH, ceil
    (7, 9, 3, 3, 2, 2, 1, 1, False), (8, 8, 2, 2, 2, 2, 0, 0, False), (9, 7, 3, 2, 2, 1, 1, 0, True),
    (10, 11, 4, 3, 3, 2, 2, 1, True), (5, 5, 2, 3, 1, 1, 1, 1, False), (6, 13, 4, 4, 4, 3, 0, 2, True),
]


@pytest.mark.parametrize("case", POOL_CASES)
def test_maxpool_bruteforce_with_ties(case):
    H, W, kW, kH, dW, dH, pW, pH, ceil = case
    rng = np.random.default_rng(8)
    x = (np.round(rng.uniform(-1, 1, (2, 3, H, W)) * 4) / 4).astype(np.float32)  # heavy ties
    y, idx = O.maxpool_updateOutput(x, kW, kH, dW, dH, pW, pH, ceil)
    ry, ridx = bf.maxpool_forward(x, kW, kH, dW, dH, pW, pH, ceil)
    assert np.array_equal(y, ry) and np.array_equal(idx, ridx)
    # index round trip: in.flat[idx - 1] == out
    flat = x.reshape(2, 3, -1)
    assert np.array_equal(np.take_along_axis(flat, (idx - 1).reshape(2, 3, -1), axis=2).reshape(y.shape), y)
    gy = rng.standard_normal(y.shape).astype(np.float32)
    close(O.maxpool_updateGradInput(x.shape, gy, idx, kW, kH, dW, dH, pW, pH, ceil), bf.maxpool_backward(x.shape, gy, idx))


def test_maxpool_dilated_bruteforce():
    rng = np.random.default_rng(9)
    x = (np.round(rng.uniform(-1, 1, (1, 2, 11, 12)) * 8) / 8).astype(np.float32)
    y, idx = O.maxpool_updateOutput(x, 3, 2, 2, 1, 1, 1, False, dilW=2, dilH=3)
    ry, ridx = bf.maxpool_forward(x, 3, 2, 2, 1, 1, 1, False, 2, 3)
    assert np.array_equal(y, ry) and np.array_equal(idx, ridx)
    gy = rng.standard_normal(y.shape).astype(np.float32)
    close(O.maxpool_updateGradInput(x.shape, gy, idx, 3, 2, 2, 1, 1, 1, False, 2, 3), bf.maxpool_backward(x.shape, gy, idx))


def test_maxpool_vs_torch_indices_on_ties():
    """CPU library indices + 1 equal the first-maximum rule on quantised input."""
    rng = np.random.default_rng(10)
    x = (np.round(rng.uniform(-1, 1, (3, 4, 30, 31)) * 64) / 64).astype(np.float32)
    for (k, s, p, ceil) in [(3, 2, 1, False), (2, 2, 0, False), (3, 2, 1, True), (4, 3, 2, True)]:
        y, idx = O.maxpool_updateOutput(x, k, k, s, s, p, p, ceil)
        ty, tidx = F.max_pool2d(torch.from_numpy(x), k, s, p, ceil_mode=ceil, return_indices=True)
        assert np.array_equal(y, ty.numpy()) and np.array_equal(idx, tidx.numpy() + 1)


def test_maxpool_nan_and_minus_inf():
    """Strict '>' against -FLT_MAX: NaN is never selected; a window holding nothing
    greater than -FLT_MAX yields value -FLT_MAX and index 0 (= -1 + base)."""
    x = np.full((1, 1, 2, 2), np.nan, np.float32)
    y, idx = O.maxpool_updateOutput(x, 2, 2, 2, 2, 0, 0, False)
    assert y[0, 0, 0, 0] == -np.finfo(np.float32).max and idx[0, 0, 0, 0] == 0
    x = np.array([[[[np.nan, 1.0], [2.0, np.nan]]]], np.float32)
    y, idx = O.maxpool_updateOutput(x, 2, 2, 2, 2, 0, 0, False)
    assert y[0, 0, 0, 0] == 2.0 and idx[0, 0, 0, 0] == 3


@pytest.mark.parametrize("case", POOL_CASES)
@pytest.mark.parametrize("include_pad", [True, False])
def test_avgpool_bruteforce(case, include_pad):
    H, W, kW, kH, dW, dH, pW, pH, ceil = case
    rng = np.random.default_rng(11)
    x = rng.standard_normal((2, 3, H, W)).astype(np.float32)
    y = O.avgpool_updateOutput(x, kW, kH, dW, dH, pW, pH, ceil, include_pad)
    ry, div = bf.avgpool_forward(x, kW, kH, dW, dH, pW, pH, ceil, include_pad)
    close(y, ry)
    gy = rng.standard_normal(y.shape).astype(np.float32)
    close(O.avgpool_updateGradInput(x.shape, gy, kW, kH, dW, dH, pW, pH, ceil, include_pad),
          bf.avgpool_backward(x.shape, gy, kW, kH, dW, dH, pW, pH, div))


def test_avgpool_vs_torch():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2, 3, 20, 22)).astype(np.float32)
    for (k, s, p, ceil, inc) in [(2, 2, 0, False, True), (3, 2, 1, False, True), (3, 2, 1, False, False), (3, 3, 1, False, False)]:
        y = O.avgpool_updateOutput(x, k, k, s, s, p, p, ceil, inc)
        tx = torch.from_numpy(x).double().requires_grad_()
        ty = F.avg_pool2d(tx, k, s, p, ceil_mode=ceil, count_include_pad=inc)
        close(y, ty.detach().numpy())
        gy = rng.standard_normal(y.shape).astype(np.float32)
        ty.backward(torch.from_numpy(gy).double())
        close(O.avgpool_updateGradInput(x.shape, gy, k, k, s, s, p, p, ceil, inc), tx.grad.numpy())


# ------------------------------------------------------------------ Threshold --
def test_threshold_vs_torch_and_special_values():
    """F.threshold + autograd fix the values on ordinary inputs; the comparison is a strict >
    (lib/THCUNN/Threshold.cu:18-21, 52-55), so the threshold itself and NaN fall to `val` / 0
    (torch's own kernels let NaN through, hence NaN is pinned here by the definition, not by torch);
    ReLU is threshold(0, 0)."""
    rng = np.random.default_rng(60)
    x = rng.standard_normal((3, 5, 7)).astype(np.float32)
    x[0, 0, :2] = [0.25, np.inf]
    for thr, val in [(0.0, 0.0), (0.25, -1.5), (-0.5, 2.0)]:
        tx = torch.from_numpy(x.copy()).requires_grad_()
        ty = F.threshold(tx, thr, val)
        y = O.threshold_updateOutput(x, thr, val)
        assert np.array_equal(y, ty.detach().numpy())
        gy = rng.standard_normal(x.shape).astype(np.float32)
        ty.backward(torch.from_numpy(gy))
        assert np.array_equal(O.threshold_updateGradInput(x, gy, thr), tx.grad.numpy())
    assert O.threshold_updateOutput(x, 0.25, -1.5)[0, 0, 0] == -1.5            # x == threshold
    xn = np.array([np.nan, 1.0], np.float32)
    assert np.array_equal(O.threshold_updateOutput(xn, 0.0, -3.0), np.array([-3.0, 1.0], np.float32))
    assert np.array_equal(O.threshold_updateGradInput(xn, np.array([5.0, 6.0], np.float32), 0.0), np.array([0.0, 6.0], np.float32))
    assert np.array_equal(O.threshold_updateOutput(x, 0, 0), np.maximum(x, 0))

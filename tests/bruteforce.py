"""Closed-form definitions of the hot-path operators as plain Python loops in
float64. Deliberately independent of oracle/: written from the mathematical
definition of each operator, not from the oracle's loop nests,
so that an indexing mistake in the oracle fails here. Tiny shapes only."""
import math

import numpy as np


def conv_out(n, k, d, p):
    return (n + 2 * p - k) // d + 1


def dw_forward(x, w, b, dW, dH, padW, padH):
    N, C, H, W = x.shape
    M, _, kH, kW = w.shape
    oH, oW = conv_out(H, kH, dH, padH), conv_out(W, kW, dW, padW)
    y = np.zeros((N, C * M, oH, oW))
    for n in range(N):
        for c in range(C):
            for j in range(M):
                for oh in range(oH):
                    for ow in range(oW):
                        s = b[j, c] if b is not None else 0.0
                        for kh in range(kH):
                            for kw in range(kW):
                                h, ww = oh * dH - padH + kh, ow * dW - padW + kw
                                if 0 <= h < H and 0 <= ww < W:
                                    s += x[n, c, h, ww] * w[j, c, kh, kw]
                        y[n, c * M + j, oh, ow] = s
    return y


def dw_grad_input(xshape, gy, w, dW, dH, padW, padH):
    N, C, H, W = xshape
    M, _, kH, kW = w.shape
    oH, oW = gy.shape[2:]
    gx = np.zeros(xshape)
    for n in range(N):
        for c in range(C):
            for j in range(M):
                for oh in range(oH):
                    for ow in range(oW):
                        for kh in range(kH):
                            for kw in range(kW):
                                h, ww = oh * dH - padH + kh, ow * dW - padW + kw
                                if 0 <= h < H and 0 <= ww < W:
                                    gx[n, c, h, ww] += gy[n, c * M + j, oh, ow] * w[j, c, kh, kw]
    return gx


def dw_grad_params(x, gy, M, kW, kH, dW, dH, padW, padH):
    N, C, H, W = x.shape
    oH, oW = gy.shape[2:]
    gw = np.zeros((M, C, kH, kW))
    gb = np.zeros((M, C))
    for n in range(N):
        for c in range(C):
            for j in range(M):
                for oh in range(oH):
                    for ow in range(oW):
                        g = gy[n, c * M + j, oh, ow]
                        gb[j, c] += g
                        for kh in range(kH):
                            for kw in range(kW):
                                h, ww = oh * dH - padH + kh, ow * dW - padW + kw
                                if 0 <= h < H and 0 <= ww < W:
                                    gw[j, c, kh, kw] += g * x[n, c, h, ww]
    return gw, gb


def conv_forward(x, w4, b, dW, dH, padW, padH):
    N, Cin, H, W = x.shape
    Cout, _, kH, kW = w4.shape
    oH, oW = conv_out(H, kH, dH, padH), conv_out(W, kW, dW, padW)
    xp = np.zeros((N, Cin, H + 2 * padH, W + 2 * padW))
    xp[:, :, padH:padH + H, padW:padW + W] = x
    y = np.zeros((N, Cout, oH, oW))
    for oh in range(oH):
        for ow in range(oW):
            patch = xp[:, :, oh * dH:oh * dH + kH, ow * dW:ow * dW + kW]
            y[:, :, oh, ow] = np.einsum("nchw,ochw->no", patch, w4)
    if b is not None:
        y += b[None, :, None, None]
    return y


def pool_out(n, k, d, p, dil, ceil_mode, any_pad):
    """Integer restatement of the float floor/ceil rule + last-window fix."""
    num = n - (dil * (k - 1) + 1) + 2 * p
    o = (-((-num) // d) if ceil_mode else num // d) + 1
    if any_pad and (o - 1) * d >= n + p:
        o -= 1
    return o


def maxpool_forward(x, kW, kH, dW, dH, padW, padH, ceil_mode, dilW=1, dilH=1):
    N, C, H, W = x.shape
    anyp = bool(padW or padH)
    oH = pool_out(H, kH, dH, padH, dilH, ceil_mode, anyp)
    oW = pool_out(W, kW, dW, padW, dilW, ceil_mode, anyp)
    y = np.zeros((N, C, oH, oW), x.dtype)
    idx = np.zeros((N, C, oH, oW), np.int64)
    fmin = -np.finfo(np.float32).max
    for n in range(N):
        for c in range(C):
            for ph in range(oH):
                for pw in range(oW):
                    best, bi = fmin, -1
                    for kh in range(kH):
                        for kw in range(kW):
                            h, w = ph * dH - padH + kh * dilH, pw * dW - padW + kw * dilW
                            if 0 <= h < H and 0 <= w < W and x[n, c, h, w] > best:
                                best, bi = x[n, c, h, w], h * W + w
                    y[n, c, ph, pw] = best
                    idx[n, c, ph, pw] = bi + 1
    return y, idx


def maxpool_backward(xshape, gy, idx):
    N, C, H, W = xshape
    gx = np.zeros(xshape)
    for n in range(N):
        for c in range(C):
            flat = gx[n, c].reshape(-1)
            for g, i in zip(gy[n, c].reshape(-1), idx[n, c].reshape(-1)):
                if i >= 1:
                    flat[i - 1] += g
    return gx


def avgpool_forward(x, kW, kH, dW, dH, padW, padH, ceil_mode, include_pad):
    N, C, H, W = x.shape
    anyp = bool(padW or padH)
    oH = pool_out(H, kH, dH, padH, 1, ceil_mode, anyp)
    oW = pool_out(W, kW, dW, padW, 1, ceil_mode, anyp)
    y = np.zeros((N, C, oH, oW))
    div = np.zeros((oH, oW))
    for ph in range(oH):
        for pw in range(oW):
            hs, ws = ph * dH - padH, pw * dW - padW
            he, we = min(hs + kH, H + padH), min(ws + kW, W + padW)
            area = (he - hs) * (we - ws)
            hs, ws, he, we = max(hs, 0), max(ws, 0), min(he, H), min(we, W)
            div[ph, pw] = area if include_pad else (he - hs) * (we - ws)
            y[:, :, ph, pw] = x[:, :, hs:he, ws:we].sum(axis=(2, 3)) / div[ph, pw]
    return y, div


def avgpool_backward(xshape, gy, kW, kH, dW, dH, padW, padH, div):
    N, C, H, W = xshape
    oH, oW = gy.shape[2:]
    gx = np.zeros(xshape)
    for ph in range(oH):
        for pw in range(oW):
            hs, ws = ph * dH - padH, pw * dW - padW
            he, we = min(hs + kH, H + padH), min(ws + kW, W + padW)
            hs, ws, he, we = max(hs, 0), max(ws, 0), min(he, H), min(we, W)
            gx[:, :, hs:he, ws:we] += (gy[:, :, ph, pw] / div[ph, pw])[:, :, None, None]
    return gx


def bn_forward(x, gamma, beta, eps):
    """Textbook training-mode batch norm over (N, spatial) per channel, float64."""
    N, C = x.shape[:2]
    xr = x.reshape(N, C, -1).astype(np.float64)
    mean = xr.mean(axis=(0, 2))
    var_b = xr.var(axis=(0, 2))
    n = xr.shape[0] * xr.shape[2]
    var_u = var_b * n / (n - 1) if n > 1 else np.full_like(var_b, np.nan)
    inv = 1.0 / np.sqrt(var_b + eps)
    g = np.ones(C) if gamma is None else gamma
    b = np.zeros(C) if beta is None else beta
    y = (xr - mean[None, :, None]) * (inv * g)[None, :, None] + b[None, :, None]
    return y.reshape(x.shape), mean, inv, var_u


def bn_backward(x, gy, gamma, mean, inv):
    N, C = x.shape[:2]
    xr = x.reshape(N, C, -1).astype(np.float64)
    gr = gy.reshape(N, C, -1).astype(np.float64)
    n = xr.shape[0] * xr.shape[2]
    g = np.ones(C) if gamma is None else gamma
    xc = xr - mean[None, :, None]
    sum_g = gr.sum(axis=(0, 2))
    dot = (gr * xc).sum(axis=(0, 2))
    gx = (gr - xc * (dot / n * inv * inv)[None, :, None] - (sum_g / n)[None, :, None]) * (inv * g)[None, :, None]
    return gx.reshape(x.shape), dot * inv, sum_g

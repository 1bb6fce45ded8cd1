#!/usr/bin/env python3
"""Writes tests/golden/thnn_golden.npz: small input/output vectors for the five
module families of the hot path.

The reference holds no stored vectors for this path (its tests compare GPU
against CPU at run time) and contains no Python, so nothing of it is imported
or executed here. Expected outputs come from PyTorch's CPU operators evaluated
in float64 - an implementation independent of both oracle/ and the HIP
kernels - with the layout conventions of the THNN entry points applied
(depthwise out-channel c*M + j, weight (M, C, kH, kW), bias (M, C); 1-based
per-plane max-pool indices; saveStd = 1/sqrt(var + eps); unbiased running
variance), plus the two known answers the reference's tests state literally
(test.lua:2597-2616).

    python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "thnn_golden.npz")
T = lambda a: torch.from_numpy(np.ascontiguousarray(a)).double()


def dw_case(rng, N, C, M, H, W, k, s, p):
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    w = rng.uniform(-0.8, 0.8, (M, C, k, k)).astype(np.float32)
    b = rng.uniform(-0.3, 0.3, (M, C)).astype(np.float32)
    tw = T(w.transpose(1, 0, 2, 3).reshape(C * M, 1, k, k)).requires_grad_()
    tb = T(b.T.reshape(C * M)).requires_grad_()
    tx = T(x).requires_grad_()
    y = F.conv2d(tx, tw, tb, stride=s, padding=p, groups=C)
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(T(gy))
    return dict(x=x, w=w, b=b, gy=gy, y=y.detach().numpy(), gx=tx.grad.numpy(),
                gw=tw.grad.numpy().reshape(C, M, k, k).transpose(1, 0, 2, 3), gb=tb.grad.numpy().reshape(C, M).T,
                geom=np.array([k, k, s, s, p, p]))


def conv_case(rng, N, Ci, Co, H, W, k, s, p):
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, k, k)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32)
    tx, tw, tb = T(x).requires_grad_(), T(w).requires_grad_(), T(b).requires_grad_()
    y = F.conv2d(tx, tw, tb, stride=s, padding=p)
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(T(gy))
    return dict(x=x, w=w.reshape(Co, -1), b=b, gy=gy, y=y.detach().numpy(), gx=tx.grad.numpy(),
                gw=tw.grad.numpy().reshape(Co, -1), gb=tb.grad.numpy(), geom=np.array([k, k, s, s, p, p]))


def bn_case(rng, shape):
    C = shape[1]
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    g = rng.random(C).astype(np.float32)
    b = rng.standard_normal(C).astype(np.float32)
    rm, rv = torch.zeros(C, dtype=torch.float64), torch.ones(C, dtype=torch.float64)
    tx, tg, tb = T(x).requires_grad_(), T(g).requires_grad_(), T(b).requires_grad_()
    y = F.batch_norm(tx, rm, rv, tg, tb, True, 0.1, 1e-5)
    gy = rng.standard_normal(shape).astype(np.float32)
    y.backward(T(gy))
    xr = T(x).reshape(shape[0], C, -1)
    mean, var = xr.mean(dim=(0, 2)), xr.var(dim=(0, 2), unbiased=False)
    y_eval = F.batch_norm(T(x), rm, rv, T(g), T(b), False, 0.1, 1e-5)
    return dict(x=x, g=g, b=b, gy=gy, y=y.detach().numpy(), gx=tx.grad.numpy(), gw=tg.grad.numpy(), gb=tb.grad.numpy(),
                save_mean=mean.numpy(), save_std=(1.0 / torch.sqrt(var + 1e-5)).numpy(), run_mean=rm.numpy(),
                run_var=rv.numpy(), y_eval=y_eval.numpy())


def pool_case(rng, N, C, H, W, k, s, p, ceil):
    x = (np.round(rng.uniform(-1, 1, (N, C, H, W)) * 16) / 16).astype(np.float32)   # ties
    tx = T(x).requires_grad_()
    y, idx = F.max_pool2d(tx, k, s, p, ceil_mode=ceil, return_indices=True)
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(T(gy))
    out = dict(x=x, gy=gy, max_y=y.detach().numpy(), max_idx=idx.numpy() + 1, max_gx=tx.grad.numpy(),
               geom=np.array([k, k, s, s, p, p, int(ceil)]))
    for inc in (True, False):
        tx2 = T(x).requires_grad_()
        ya = F.avg_pool2d(tx2, k, s, p, ceil_mode=ceil, count_include_pad=inc)
        assert tuple(ya.shape) == tuple(y.shape)
        ya.backward(T(gy))
        out[f"avg_y_{int(inc)}"] = ya.detach().numpy()
        out[f"avg_gx_{int(inc)}"] = tx2.grad.numpy()
    return out


def dilpool_case(rng, N, C, H, W, k, s, p, dil, ceil):
    x = (np.round(rng.uniform(-1, 1, (N, C, H, W)) * 16) / 16).astype(np.float32)   # ties
    tx = T(x).requires_grad_()
    y, idx = F.max_pool2d(tx, k, s, p, dilation=dil, ceil_mode=ceil, return_indices=True)
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(T(gy))
    return dict(x=x, gy=gy, max_y=y.detach().numpy(), max_idx=idx.numpy() + 1, max_gx=tx.grad.numpy(),
                geom=np.array([k, k, s, s, p, p, dil, dil, int(ceil)]))


def dilconv_case(rng, N, Ci, Co, H, W, k, s, p, dil):
    """SpatialDilatedConvolution: 4-D weight (Cout, Cin, kH, kW)."""
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, k, k)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32)
    tx, tw, tb = T(x).requires_grad_(), T(w).requires_grad_(), T(b).requires_grad_()
    y = F.conv2d(tx, tw, tb, stride=s, padding=p, dilation=dil)
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(T(gy))
    return dict(x=x, w=w, b=b, gy=gy, y=y.detach().numpy(), gx=tx.grad.numpy(), gw=tw.grad.numpy(), gb=tb.grad.numpy(),
                geom=np.array([k, k, s, s, p, p, dil, dil]))


def fullconv_case(rng, N, Ci, Co, H, W, k, s, p, adj):
    """SpatialFullConvolution: weight (Cin, Cout, kH, kW), output (H - 1) s - 2 p + k + adj."""
    x = rng.standard_normal((N, Ci, H, W)).astype(np.float32)
    w = (rng.standard_normal((Ci, Co, k, k)) * 0.2).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32)
    tx, tw, tb = T(x).requires_grad_(), T(w).requires_grad_(), T(b).requires_grad_()
    y = F.conv_transpose2d(tx, tw, tb, stride=s, padding=p, output_padding=adj)
    gy = rng.standard_normal(tuple(y.shape)).astype(np.float32)
    y.backward(T(gy))
    return dict(x=x, w=w, b=b, gy=gy, y=y.detach().numpy(), gx=tx.grad.numpy(), gw=tw.grad.numpy(), gb=tb.grad.numpy(),
                geom=np.array([k, k, s, s, p, p, adj, adj]))


def threshold_case(rng, shape, th, val):
    """Threshold: y = x > th ? x : val; gradInput = x > th ? gradOutput : 0 (lib/THCUNN/Threshold.cu). Values
    quantised so that some inputs equal the threshold exactly (the comparison is strict)."""
    x = (np.round(rng.standard_normal(shape) * 4) / 4).astype(np.float32)
    gy = rng.standard_normal(shape).astype(np.float32)
    y = np.where(x > np.float32(th), x, np.float32(val)).astype(np.float32)
    gx = np.where(x > np.float32(th), gy, np.float32(0)).astype(np.float32)
    return dict(x=x, gy=gy, y=y, gx=gx, param=np.array([th, val], np.float32))


def bnrelu_case(rng, shape):
    """BatchNormalization (train) followed by Threshold(0, 0): activation, and the gradients of the pair."""
    C = shape[1]
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    g = (rng.random(C) + 0.25).astype(np.float32)
    b = rng.standard_normal(C).astype(np.float32)
    rm, rv = torch.zeros(C, dtype=torch.float64), torch.ones(C, dtype=torch.float64)
    tx, tg, tb = T(x).requires_grad_(), T(g).requires_grad_(), T(b).requires_grad_()
    a = F.relu(F.batch_norm(tx, rm, rv, tg, tb, True, 0.1, 1e-5))
    ga = rng.standard_normal(shape).astype(np.float32)
    a.backward(T(ga))
    return dict(x=x, g=g, b=b, ga=ga, a=a.detach().numpy(), gx=tx.grad.numpy(), gw=tg.grad.numpy(), gb=tb.grad.numpy())


def main():
    rng = np.random.default_rng(20240601)
    cases = {
        "dw_ref_shape": dw_case(rng, 3, 3, 4, 28, 28, 3, 1, 1),       # the reference test's geometry (test.lua:6639-6645)
        "dw_s2": dw_case(rng, 2, 8, 1, 24, 24, 3, 2, 1),
        "dw_k5": dw_case(rng, 2, 3, 2, 16, 20, 5, 1, 2),
        "conv_3x3": conv_case(rng, 2, 8, 16, 12, 12, 3, 1, 1),
        "conv_s2": conv_case(rng, 3, 5, 12, 15, 13, 3, 2, 0),
        "bn_4d": bn_case(rng, (6, 5, 7, 9)),
        "bn_2d": bn_case(rng, (16, 7)),
        "pool_3s2p1": pool_case(rng, 2, 3, 24, 24, 3, 2, 1, False),
        "pool_2s2": pool_case(rng, 2, 3, 24, 24, 2, 2, 0, False),
        "pool_3s2p1_ceil": pool_case(rng, 1, 2, 15, 18, 3, 2, 1, True),     # ceil mode adds a last, clipped window: 8x10 outputs
        # ceil mode where the last window would start in the padding and is dropped again
        # (lib/THCUNN/generic/SpatialDilatedMaxPooling.cu:56-64): 7 -> 4 and 9 -> 5 outputs instead of 5 and 6
        "pool_2s2p1_ceil_drop": pool_case(rng, 2, 3, 7, 9, 2, 2, 1, True),
    }
    # cases added later draw from a generator of their own, so that the vectors above stay bit for bit what they were
    rng2 = np.random.default_rng(20240602)
    cases.update({
        "pool_dil2": dilpool_case(rng2, 2, 3, 13, 14, 3, 2, 1, 2, False),
        "dilconv_d2": dilconv_case(rng2, 2, 4, 6, 12, 11, 3, 1, 2, 2),
        "fullconv_s2": fullconv_case(rng2, 2, 6, 4, 7, 8, 4, 2, 1, 0),
        "thr": threshold_case(rng2, (3, 5, 7, 6), 0.25, -0.5),
        "bnrelu_4d": bnrelu_case(rng2, (6, 5, 7, 9)),
    })
    flat = {}
    for cname, d in cases.items():
        for k, v in d.items():
            v = np.asarray(v)
            flat[f"{cname}/{k}"] = v.astype(np.float32) if v.dtype == np.float64 else v
    # known answers written out in the reference's own test (test.lua:2597-2616)
    flat["kat_avgpool/x"] = np.full((1, 1, 1, 1), 3.0, np.float32)
    flat["kat_avgpool/exclude_pad"] = np.float32(3.0)
    flat["kat_avgpool/include_pad"] = np.float32(0.75)
    np.savez_compressed(OUT, **flat)
    print(f"wrote {OUT}: {len(flat)} arrays, {os.path.getsize(OUT) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()

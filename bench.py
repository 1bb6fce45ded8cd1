#!/usr/bin/env python3
"""Benchmark of the THCUNN spatial-conv hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2] [--all]

A step is one pass of the workload's entry points over one synthetic batch,
called through the C ABI of libTHCUNN.so. The default workload is the one the
headline metric is quoted on: SpatialDepthWiseConvolution forward +
updateGradInput + accGradParameters, fp32, N=64 C=128 56x56 -> 28x28, 3x3
stride 2 pad 1 (the MobileNet stride-2 layer). Inputs live in HBM before the timed
region; four buffer sets are rotated so that no step finds its inputs in the
256 MB Infinity Cache from the step before.

Prints ONE JSON line: images/s for the whole job (K steps between two
synchronisations, nothing but the entry-point calls on the stream), plus
  roofline     - the dominant entry point's algorithmic bytes (or flops) per launch
                 over its average duration measured with HIP events on the
                 stream the kernels run on, over the same K steps run a second
                 time with that entry point bracketed, against MI355X's published
                 peak (median, min and the whole step's fraction beside it);
                 roofline.cold: the same figures when the entry points of a step
                 work on different buffer sets, so that no call finds in the
                 Infinity Cache what an earlier call of the step touched;
                 roofline.copy_gbs: what a plain 128 MiB copy reaches in this run;
  cpu_baseline - the CPU oracle (a port of the reference algorithm) timed on
                 this host's cores on a bounded sample of the same workload;
  workloads    - with --all, the same figures for the other four configurations.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
FP32_MFMA_PEAK_TFLOPS = 157.3
METRIC = "DW-conv fwd+bwd images/s + achieved HBM GB/s (% of peak), 1 MI355X"

# HBM bytes per entry-point call, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch) and kept
# beside the summaries they come from: profiles/hbm_traffic_table.txt has one row per kernel of an entry point with the
# raw counter averages, the summary file and the commit the counters were collected at. Scale factors from the copy
# kernel of known size: FETCH_SIZE x 2, WRITE_SIZE x 1.
_KIB = 1024
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic_table.txt")


def load_traffic(path=TRAFFIC_TABLE):
    """{(workload, entry point): dict(bytes=..., source=..., commit=...)}; empty when the table is missing."""
    out = {}
    if not os.path.exists(path):
        return out
    for line in open(path):
        line = line.split("#", 1)[0].split()
        if len(line) != 7:
            continue
        wl, entry, _kernel, fetch, write, source, commit = line
        e = out.setdefault((wl, entry), dict(bytes=0, source=source, commit=commit))
        e["bytes"] += int((float(fetch) * 2.0 + float(write)) * _KIB)
    return out


class Hip:
    def __init__(self):
        self.lib = C.CDLL("libamdhip64.so")
        self.lib.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.lib.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.lib.hipEventSynchronize.argtypes = [C.c_void_p]
        self.lib.hipStreamQuery.argtypes = [C.c_void_p]

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError(f"{what} failed with hipError {rc}")

    def event(self):
        # hipEventDisableSystemFence: the record does not flush the caches to system
        # scope, so bracketing a kernel costs ~1 us of dispatch instead of ~3 us
        e = C.c_void_p()
        self.check(self.lib.hipEventCreateWithFlags(C.byref(e), 0x20000000), "hipEventCreateWithFlags")
        return e

    def record(self, e, stream):
        self.check(self.lib.hipEventRecord(e, stream), "hipEventRecord")

    def elapsed_ms(self, a, b):
        self.check(self.lib.hipEventSynchronize(b), "hipEventSynchronize")
        ms = C.c_float()
        self.check(self.lib.hipEventElapsedTime(C.byref(ms), a, b), "hipEventElapsedTime")
        return float(ms.value)

    def sync(self, stream=None):
        # With a stream: poll it until it has drained instead of sleeping in the runtime - the wake-up after a
        # blocking wait costs tens of microseconds, a sizeable part of a 20-step timed region of 1.4 ms.
        if stream is not None:
            while True:
                rc = self.lib.hipStreamQuery(stream)
                if rc == 0:
                    break
                if rc != 600:  # hipErrorNotReady
                    self.check(rc, "hipStreamQuery")
        self.check(self.lib.hipDeviceSynchronize(), "hipDeviceSynchronize")


# --------------------------------------------------------------- workloads ----
# Each workload builds `nsets` independent buffer sets and returns
#   calls(set_index) -> list of (kernel_name, fn)       the step, in order
#   work              -> {kernel_name: (amount, "bytes"|"flops")} algorithmic work per launch
#   images            -> batch size
#   cpu(sample)       -> (seconds, images) of the oracle on a bounded sample

def _kaiming_uniform(rng, shape, fan_in):
    b = np.sqrt(6.0 / fan_in)
    return rng.uniform(-b, b, shape).astype(np.float32)


def wl_dw(cfg, nsets):
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    if cfg == "cfg1":
        N, Cc, H, k, s, p, seed, full = 32, 32, 112, 3, 1, 1, 0, False
    elif cfg == "dw147":  # a plane width that is not a multiple of 4 (Xception entry flow): bands of rows per workgroup
        N, Cc, H, k, s, p, seed, full = 32, 128, 147, 3, 1, 1, 5, True
    elif cfg == "dw14":   # small planes (MobileNet 14x14 stage): several planes per workgroup
        N, Cc, H, k, s, p, seed, full = 64, 512, 14, 3, 1, 1, 6, True
    else:
        N, Cc, H, k, s, p, seed, full = 64, 128, 56, 3, 2, 1, 1, True
    oH = (H + 2 * p - k) // s + 1
    rng = np.random.default_rng(seed)
    x = (rng.uniform(-1, 1, (N, Cc, H, H)) if cfg == "cfg1" else rng.standard_normal((N, Cc, H, H))).astype(np.float32)
    w = _kaiming_uniform(rng, (1, Cc, k, k), k * k)
    b = rng.uniform(-1 / 3, 1 / 3, (1, Cc)).astype(np.float32)
    gy = rng.standard_normal((N, Cc, oH, oH)).astype(np.float32)
    sets = []
    for _ in range(nsets):
        sets.append(dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), gx=CT(), w=CT.from_numpy(w),
                         b=CT.from_numpy(b), gw=CT.from_numpy(np.zeros_like(w)), gb=CT.from_numpy(np.zeros_like(b)),
                         cols=CT(), ones=CT()))
    xb, yb = x.nbytes, gy.nbytes

    def calls(i):
        t = sets[i]
        g = (k, k, s, s, p, p)
        fwd = ("dw_updateOutput", lambda: THNN.SpatialDepthWiseConvolution_updateOutput(
            t["x"], t["y"], t["w"], t["b"], t["cols"], t["ones"], *g))
        if not full:
            return [fwd]
        return [fwd,
                ("dw_updateGradInput", lambda: THNN.SpatialDepthWiseConvolution_updateGradInput(
                    t["x"], t["gy"], t["gx"], t["w"], t["cols"], t["ones"], *g)),
                ("dw_accGradParameters", lambda: THNN.SpatialDepthWiseConvolution_accGradParameters(
                    t["x"], t["gy"], t["gw"], t["gb"], t["cols"], t["ones"], *g, 1.0))]

    work = {"dw_updateOutput": (xb + yb, "bytes"), "dw_updateGradInput": (xb + yb, "bytes"),
            "dw_accGradParameters": (xb + yb, "bytes")}

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            O.dwconv_updateOutput(x, w, b, k, k, s, s, p, p)
            if full:
                O.dwconv_updateGradInput(x.shape, gy, w, k, k, s, s, p, p)
                O.dwconv_accGradParameters(x, gy, np.zeros_like(w), np.zeros_like(b), k, k, s, s, p, p, 1.0)
        return time.perf_counter() - t0, reps * N, f"{reps} full passes of {cfg} ({N} images each)"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        np.testing.assert_allclose(t["y"].numpy(), O.dwconv_updateOutput(x, w, b, k, k, s, s, p, p), rtol=1e-5, atol=1e-4)
        if full:
            np.testing.assert_allclose(t["gx"].numpy(), O.dwconv_updateGradInput(x.shape, gy, w, k, k, s, s, p, p),
                                       rtol=1e-5, atol=1e-4)
            rgw, rgb = O.dwconv_accGradParameters(x, gy, np.zeros_like(w), np.zeros_like(b), k, k, s, s, p, p, 1.0)
            np.testing.assert_allclose(t["gw"].numpy(), rgw, rtol=1e-3, atol=1e-3)
            np.testing.assert_allclose(t["gb"].numpy(), rgb, rtol=1e-3, atol=1e-3)
            t["gw"].fill(0.0), t["gb"].fill(0.0)

    desc = (f"SpatialDepthWiseConvolution {'fwd+gradInput+accGradParameters' if full else 'fwd'} fp32 "
            f"N={N} C={Cc} {H}x{H}->{oH}x{oH} k{k} s{s} p{p} M=1")
    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, desc=desc, bound="hbm")


def wl_bn(nsets):
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    N, Cc, H = 64, 256, 28
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((N, Cc, H, H)) * 2 + 0.5).astype(np.float32)
    gy = rng.standard_normal((N, Cc, H, H)).astype(np.float32)
    g = rng.random(Cc).astype(np.float32)
    b = np.zeros(Cc, np.float32)
    sets = []
    for _ in range(nsets):
        sets.append(dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), gx=CT.with_size(N, Cc, H, H), g=CT.from_numpy(g),
                         b=CT.from_numpy(b), rm=CT.from_numpy(np.zeros(Cc, np.float32)),
                         rv=CT.from_numpy(np.ones(Cc, np.float32)), sm=CT.with_size(Cc), ss=CT.with_size(Cc),
                         gw=CT.from_numpy(np.zeros(Cc, np.float32)), gb=CT.from_numpy(np.zeros(Cc, np.float32))))

    def calls(i):
        t = sets[i]
        return [("bn_updateOutput", lambda: THNN.BatchNormalization_updateOutput(
                    t["x"], t["y"], t["g"], t["b"], t["rm"], t["rv"], t["sm"], t["ss"], True, 0.1, 1e-5)),
                ("bn_backward", lambda: THNN.BatchNormalization_backward(
                    t["x"], t["gy"], t["gx"], t["gw"], t["gb"], t["g"], t["rm"], t["rv"], t["sm"], t["ss"], True, 1.0, 1e-5))]

    work = {"bn_updateOutput": (2 * x.nbytes, "bytes"), "bn_backward": (3 * x.nbytes, "bytes")}

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            rm, rv = np.zeros(Cc, np.float32), np.ones(Cc, np.float32)
            _, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, 0.1, 1e-5)
            O.bn_backward(x, gy, g, rm, rv, sm, ss, True, 1.0, 1e-5, np.zeros(Cc, np.float32), np.zeros(Cc, np.float32))
        return time.perf_counter() - t0, reps * N, f"{reps} full passes of cfg3 ({N} images each)"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        rm, rv = np.zeros(Cc, np.float32), np.ones(Cc, np.float32)
        ry, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, 0.1, 1e-5)
        np.testing.assert_allclose(t["y"].numpy(), ry, rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["ss"].numpy(), ss, rtol=1e-3)
        rgi, rgw, _ = O.bn_backward(x, gy, g, rm, rv, sm, ss, True, 1.0, 1e-5, np.zeros(Cc, np.float32), np.zeros(Cc, np.float32))
        np.testing.assert_allclose(t["gx"].numpy(), rgi, rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["gw"].numpy(), rgw, rtol=1e-3, atol=1e-2)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="hbm",
                desc=f"SpatialBatchNormalization train fwd+bwd fp32 N={N} C={Cc} {H}x{H} affine eps=1e-5 momentum=0.1")


def wl_pool(nsets, odd=False):
    from cunn_amd import CudaLongTensor as LT, CudaTensor as CT, THNN
    from oracle import oracle as O
    # odd: 71x71 planes (Inception-style 3x3 stride-2 max pooling without padding, 3x3 stride-1 average pooling)
    N, Cc, H = (32, 192, 71) if odd else (64, 64, 112)
    mk, ms, mp = (3, 2, 0) if odd else (3, 2, 1)
    ak, as_, ap_ = (3, 1, 1) if odd else (2, 2, 0)
    oM, oA = (H + 2 * mp - mk) // ms + 1, (H + 2 * ap_ - ak) // as_ + 1
    rng = np.random.default_rng(7 if odd else 3)
    x = (np.round(rng.uniform(-1, 1, (N, Cc, H, H)) * 64) / 64).astype(np.float32)
    gy = rng.standard_normal((N, Cc, oM, oM)).astype(np.float32)
    gya = gy if oA == oM else rng.standard_normal((N, Cc, oA, oA)).astype(np.float32)
    sets = []
    for _ in range(nsets):
        sets.append(dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), gya=CT.from_numpy(gya), y=CT(), idx=LT(), gx=CT(), ya=CT(),
                         gxa=CT()))
    M, A = (mk, mk, ms, ms, mp, mp, False), (ak, ak, as_, as_, ap_, ap_, False, True)

    def calls(i):
        t = sets[i]
        return [("maxpool_updateOutput", lambda: THNN.SpatialMaxPooling_updateOutput(t["x"], t["y"], t["idx"], *M)),
                ("maxpool_updateGradInput", lambda: THNN.SpatialMaxPooling_updateGradInput(t["x"], t["gy"], t["gx"], t["idx"], *M)),
                ("avgpool_updateOutput", lambda: THNN.SpatialAveragePooling_updateOutput(t["x"], t["ya"], *A)),
                ("avgpool_updateGradInput", lambda: THNN.SpatialAveragePooling_updateGradInput(t["x"], t["gya"], t["gxa"], *A))]

    xb, yb, yab = x.nbytes, gy.nbytes, gya.nbytes
    work = {"maxpool_updateOutput": (xb + yb + 2 * yb, "bytes"), "maxpool_updateGradInput": (yb + 2 * yb + xb, "bytes"),
            "avgpool_updateOutput": (xb + yab, "bytes"), "avgpool_updateGradInput": (yab + xb, "bytes")}

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            _, idx = O.maxpool_updateOutput(x, *M)
            O.maxpool_updateGradInput(x.shape, gy, idx, *M)
            O.avgpool_updateOutput(x, *A)
            O.avgpool_updateGradInput(x.shape, gya, *A)
        return time.perf_counter() - t0, reps * N, f"{reps} full passes of {'pool71' if odd else 'cfg4'} ({N} images each)"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        ry, ridx = O.maxpool_updateOutput(x, *M)
        assert np.array_equal(t["y"].numpy(), ry) and np.array_equal(t["idx"].numpy(), ridx)
        np.testing.assert_allclose(t["gx"].numpy(), O.maxpool_updateGradInput(x.shape, gy, ridx, *M), rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["ya"].numpy(), O.avgpool_updateOutput(x, *A), rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["gxa"].numpy(), O.avgpool_updateGradInput(x.shape, gya, *A), rtol=1e-5, atol=1e-4)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="hbm",
                desc=f"SpatialMaxPooling {mk}x{mk} s{ms} p{mp} (+indices) and SpatialAveragePooling {ak}x{ak} s{as_} p{ap_}, fwd+bwd fp32 "
                     f"N={N} C={Cc} {H}x{H}->{oM}x{oM} / {oA}x{oA}")


def wl_conv(nsets, pointwise=False, first=False):
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    # pointwise: the 1x1 convolution behind the metric's depthwise layer in MobileNet-v1 (128 -> 128 at 56 x 56)
    # first: the first layer of ResNet (3 -> 64 planes, 7x7 stride 2 at 224 x 224)
    N, Ci, Co, H, k, st = (64, 128, 128, 56, 1, 1) if pointwise else (32, 3, 64, 224, 7, 2) if first else (64, 256, 256, 28, 3, 1)
    K = Ci * k * k
    oH = (H + 2 * (k // 2) - k) // st + 1
    rng = np.random.default_rng(4)
    x = rng.standard_normal((N, Ci, H, H)).astype(np.float32)
    gy = rng.standard_normal((N, Co, oH, oH)).astype(np.float32)
    w = (rng.standard_normal((Co, K)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.uniform(-0.02, 0.02, Co).astype(np.float32)
    sets = []
    for _ in range(nsets):
        sets.append(dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), gx=CT(), w=CT.from_numpy(w), b=CT.from_numpy(b),
                         gw=CT.from_numpy(np.zeros_like(w)), gb=CT.from_numpy(np.zeros_like(b)), cols=CT(), gcols=CT(), ones=CT()))
    g = (k, k, st, st, k // 2, k // 2)

    def calls(i):
        t = sets[i]
        return [("convmm_updateOutput", lambda: THNN.SpatialConvolutionMM_updateOutput(t["x"], t["y"], t["w"], t["b"], t["cols"], t["ones"], *g)),
                ("convmm_updateGradInput", lambda: THNN.SpatialConvolutionMM_updateGradInput(t["x"], t["gy"], t["gx"], t["w"], t["gcols"], t["ones"], *g)),
                ("convmm_accGradParameters", lambda: THNN.SpatialConvolutionMM_accGradParameters(t["x"], t["gy"], t["gw"], t["gb"], t["cols"], t["ones"], *g, 1.0))]

    fl = 2.0 * Co * K * oH * oH * N
    work = {"convmm_updateOutput": (fl, "flops"), "convmm_updateGradInput": (fl, "flops"), "convmm_accGradParameters": (fl, "flops")}
    ns = 4  # images of the CPU sample

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            O.convmm_updateOutput(x[:ns], w, b, *g)
            O.convmm_updateGradInput((ns,) + x.shape[1:], gy[:ns], w, *g)
            O.convmm_accGradParameters(x[:ns], gy[:ns], np.zeros_like(w), np.zeros_like(b), *g, 1.0)
        return time.perf_counter() - t0, reps * ns, f"{reps} passes over the first {ns} of {N} images"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        m = 2  # images checked against the oracle
        np.testing.assert_allclose(t["y"].numpy()[:m], O.convmm_updateOutput(x[:m], w, b, *g), rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["gx"].numpy()[:m], O.convmm_updateGradInput((m,) + x.shape[1:], gy[:m], w, *g), rtol=1e-5, atol=1e-4)
        t["gw"].fill(0.0), t["gb"].fill(0.0)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="mfma",
                desc=f"SpatialConvolutionMM fwd+gradInput+accGradParameters fp32 N={N} Cin={Ci} Cout={Co} {H}x{H} k{k} s{st} p{k // 2} bias")


def wl_dilconv(nsets):
    """Beyond the five configurations: SpatialDilatedConvolution at the cfg5 shape with dilation 2 ("same" padding 2)."""
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    N, Ci, Co, H, k, dil = 64, 256, 256, 28, 3, 2
    K = Ci * k * k
    rng = np.random.default_rng(5)
    x = rng.standard_normal((N, Ci, H, H)).astype(np.float32)
    gy = rng.standard_normal((N, Co, H, H)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, k, k)) * np.sqrt(2.0 / K)).astype(np.float32)
    b = rng.uniform(-0.02, 0.02, Co).astype(np.float32)
    sets = [dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), gx=CT(), w=CT.from_numpy(w), b=CT.from_numpy(b),
                 gw=CT.from_numpy(np.zeros_like(w)), gb=CT.from_numpy(np.zeros_like(b)), cols=CT(), gcols=CT(), ones=CT())
            for _ in range(nsets)]
    g = (k, k, 1, 1, dil, dil, dil, dil)

    def calls(i):
        t = sets[i]
        return [("dilconv_updateOutput", lambda: THNN.SpatialDilatedConvolution_updateOutput(t["x"], t["y"], t["w"], t["b"], t["cols"], t["ones"], *g)),
                ("dilconv_updateGradInput", lambda: THNN.SpatialDilatedConvolution_updateGradInput(t["x"], t["gy"], t["gx"], t["w"], t["gcols"], *g)),
                ("dilconv_accGradParameters", lambda: THNN.SpatialDilatedConvolution_accGradParameters(t["x"], t["gy"], t["gw"], t["gb"], t["cols"], t["ones"], *g, 1.0))]

    fl = 2.0 * Co * K * H * H * N
    work = {"dilconv_updateOutput": (fl, "flops"), "dilconv_updateGradInput": (fl, "flops"), "dilconv_accGradParameters": (fl, "flops")}
    ns = 4

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            O.dilconv_updateOutput(x[:ns], w, b, *g)
            O.dilconv_updateGradInput((ns,) + x.shape[1:], gy[:ns], w, *g)
            O.dilconv_accGradParameters(x[:ns], gy[:ns], np.zeros((Co, K), np.float32), np.zeros_like(b), *g, 1.0)
        return time.perf_counter() - t0, reps * ns, f"{reps} passes over the first {ns} of {N} images"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        m = 2
        np.testing.assert_allclose(t["y"].numpy()[:m], O.dilconv_updateOutput(x[:m], w, b, *g), rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["gx"].numpy()[:m], O.dilconv_updateGradInput((m,) + x.shape[1:], gy[:m], w, *g), rtol=1e-5, atol=1e-4)
        t["gw"].fill(0.0), t["gb"].fill(0.0)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="mfma",
                desc=f"SpatialDilatedConvolution fwd+gradInput+accGradParameters fp32 N={N} Cin={Ci} Cout={Co} {H}x{H} k3 s1 p2 dilation 2 bias")


def wl_fullconv(nsets):
    """Beyond the five configurations: SpatialFullConvolution, the 2x upsampling transposed convolution of a decoder."""
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    N, Ci, Co, H, k = 64, 256, 128, 14, 4
    rng = np.random.default_rng(6)
    oH = (H - 1) * 2 - 2 + k
    x = rng.standard_normal((N, Ci, H, H)).astype(np.float32)
    gy = rng.standard_normal((N, Co, oH, oH)).astype(np.float32)
    w = (rng.standard_normal((Ci, Co, k, k)) * np.sqrt(2.0 / (Ci * k * k))).astype(np.float32)
    b = rng.uniform(-0.02, 0.02, Co).astype(np.float32)
    sets = [dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), gx=CT(), w=CT.from_numpy(w), b=CT.from_numpy(b),
                 gw=CT.from_numpy(np.zeros_like(w)), gb=CT.from_numpy(np.zeros_like(b)), cols=CT(), gcols=CT(), ones=CT())
            for _ in range(nsets)]
    g = (k, k, 2, 2, 1, 1, 0, 0)
    og = (k, k, 2, 2, 1, 1, 1, 1, 0, 0)

    def calls(i):
        t = sets[i]
        return [("fullconv_updateOutput", lambda: THNN.SpatialFullConvolution_updateOutput(t["x"], t["y"], t["w"], t["b"], t["cols"], t["ones"], *g)),
                ("fullconv_updateGradInput", lambda: THNN.SpatialFullConvolution_updateGradInput(t["x"], t["gy"], t["gx"], t["w"], t["gcols"], *g)),
                ("fullconv_accGradParameters", lambda: THNN.SpatialFullConvolution_accGradParameters(t["x"], t["gy"], t["gw"], t["gb"], t["cols"], t["ones"], *g, 1.0))]

    fl = 2.0 * Ci * Co * k * k * H * H * N   # every input pixel meets every tap of every (Cin, Cout) pair once
    work = {"fullconv_updateOutput": (fl, "flops"), "fullconv_updateGradInput": (fl, "flops"), "fullconv_accGradParameters": (fl, "flops")}
    ns = 4

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            O.fullconv_updateOutput(x[:ns], w, b, *og)
            O.fullconv_updateGradInput((ns,) + x.shape[1:], gy[:ns], w, *og)
            O.fullconv_accGradParameters(x[:ns], gy[:ns], np.zeros_like(w), np.zeros_like(b), *og, scale=1.0)
        return time.perf_counter() - t0, reps * ns, f"{reps} passes over the first {ns} of {N} images"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        m = 2
        np.testing.assert_allclose(t["y"].numpy()[:m], O.fullconv_updateOutput(x[:m], w, b, *og), rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(t["gx"].numpy()[:m], O.fullconv_updateGradInput((m,) + x.shape[1:], gy[:m], w, *og), rtol=1e-5, atol=1e-4)
        t["gw"].fill(0.0), t["gb"].fill(0.0)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="mfma",
                desc=f"SpatialFullConvolution fwd+gradInput+accGradParameters fp32 N={N} Cin={Ci} Cout={Co} {H}x{H}->{oH}x{oH} k4 s2 p1 bias")


def wl_relu(nsets):
    """Beyond the five configurations: Threshold (ReLU) forward + backward on the cfg2 activation tensor."""
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    shape = (64, 128, 56, 56)
    rng = np.random.default_rng(7)
    x = rng.standard_normal(shape).astype(np.float32)
    gy = rng.standard_normal(shape).astype(np.float32)
    sets = [dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), gx=CT()) for _ in range(nsets)]

    def calls(i):
        t = sets[i]
        return [("threshold_updateOutput", lambda: THNN.Threshold_updateOutput(t["x"], t["y"], 0.0, 0.0, False)),
                ("threshold_updateGradInput", lambda: THNN.Threshold_updateGradInput(t["x"], t["gy"], t["gx"], 0.0, 0.0, False))]

    work = {"threshold_updateOutput": (2 * x.nbytes, "bytes"), "threshold_updateGradInput": (3 * x.nbytes, "bytes")}

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            O.threshold_updateOutput(x, 0.0, 0.0)
            O.threshold_updateGradInput(x, gy, 0.0)
        return time.perf_counter() - t0, reps * shape[0], f"{reps} full passes ({shape[0]} images each), numpy"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        assert np.array_equal(t["y"].numpy(), O.threshold_updateOutput(x, 0.0, 0.0))
        assert np.array_equal(t["gx"].numpy(), O.threshold_updateGradInput(x, gy, 0.0))

    return dict(calls=calls, work=work, images=shape[0], cpu=cpu, verify=verify, bound="hbm",
                desc="Threshold (ReLU) fwd+bwd fp32 N=64 C=128 56x56")


def wl_bnrelu(nsets, fused=True):
    """Beyond the five configurations: BatchNormalization (train) + ReLU forward and backward on the cfg3 tensor, as the
    fused entry points (include/THCUNN_fused.h) or as the four separate calls they replace."""
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    N, Cc, H = 64, 256, 28
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((N, Cc, H, H)) * 2 + 0.5).astype(np.float32)
    gy = rng.standard_normal((N, Cc, H, H)).astype(np.float32)
    g = (rng.random(Cc) + 0.25).astype(np.float32)
    b = rng.standard_normal(Cc).astype(np.float32)
    z = lambda: CT.from_numpy(np.zeros(Cc, np.float32))
    sets = [dict(x=CT.from_numpy(x), gy=CT.from_numpy(gy), y=CT(), a=CT(), ga=CT(), gx=CT.with_size(N, Cc, H, H), g=CT.from_numpy(g),
                 b=CT.from_numpy(b), rm=z(), rv=CT.from_numpy(np.ones(Cc, np.float32)), sm=CT.with_size(Cc), ss=CT.with_size(Cc),
                 gw=z(), gb=z()) for _ in range(nsets)]

    def calls(i):
        t = sets[i]
        if fused:
            return [("bnrelu_updateOutput", lambda: THNN.BatchNormalizationReLU_updateOutput(
                        t["x"], t["a"], t["g"], t["b"], t["rm"], t["rv"], t["sm"], t["ss"], True, 0.1, 1e-5)),
                    ("bnrelu_backward", lambda: THNN.BatchNormalizationReLU_backward(
                        t["x"], t["gy"], t["gx"], t["gw"], t["gb"], t["g"], t["b"], t["rm"], t["rv"], t["sm"], t["ss"], True, 1.0, 1e-5))]
        return [("bn_updateOutput", lambda: THNN.BatchNormalization_updateOutput(
                    t["x"], t["y"], t["g"], t["b"], t["rm"], t["rv"], t["sm"], t["ss"], True, 0.1, 1e-5)),
                ("threshold_updateOutput", lambda: THNN.Threshold_updateOutput(t["y"], t["a"], 0.0, 0.0, False)),
                ("threshold_updateGradInput", lambda: THNN.Threshold_updateGradInput(t["y"], t["gy"], t["ga"], 0.0, 0.0, False)),
                ("bn_backward", lambda: THNN.BatchNormalization_backward(
                    t["x"], t["ga"], t["gx"], t["gw"], t["gb"], t["g"], t["rm"], t["rv"], t["sm"], t["ss"], True, 1.0, 1e-5))]

    xb = x.nbytes
    # algorithmic bytes of the pair: x in, activation out; x and gradOutput in, gradInput out - whichever way it is computed
    work = ({"bnrelu_updateOutput": (2 * xb, "bytes"), "bnrelu_backward": (3 * xb, "bytes")} if fused else
            {"bn_updateOutput": (2 * xb, "bytes"), "threshold_updateOutput": (0, "bytes"), "threshold_updateGradInput": (0, "bytes"),
             "bn_backward": (3 * xb, "bytes")})

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            rm, rv = np.zeros(Cc, np.float32), np.ones(Cc, np.float32)
            y, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, 0.1, 1e-5)
            O.threshold_updateOutput(y, 0.0, 0.0)
            O.bn_backward(x, O.threshold_updateGradInput(y, gy, 0.0), g, rm, rv, sm, ss, True, 1.0, 1e-5,
                          np.zeros(Cc, np.float32), np.zeros(Cc, np.float32))
        return time.perf_counter() - t0, reps * N, f"{reps} full passes ({N} images each)"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        rm, rv = np.zeros(Cc, np.float32), np.ones(Cc, np.float32)
        y, sm, ss = O.bn_updateOutput(x, g, b, rm, rv, True, 0.1, 1e-5)
        np.testing.assert_allclose(t["a"].numpy(), O.threshold_updateOutput(y, 0.0, 0.0), rtol=1e-5, atol=1e-4)
        t["gw"].fill(0.0), t["gb"].fill(0.0)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="hbm",
                desc=f"BatchNormalization (train) + ReLU fwd+bwd fp32 N={N} C={Cc} {H}x{H}, "
                     + ("fused entry points" if fused else "four separate calls"))


def wl_convrelu(nsets, fused=True):
    """Beyond the five configurations: a 1x1 convolution (128 -> 128 planes at 56 x 56, N = 64) followed by ReLU, forward,
    as the fused entry point (include/THCUNN_fused.h) or as the two calls it replaces."""
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    N, Ci, Co, H = 64, 128, 128, 56
    rng = np.random.default_rng(9)
    x = rng.standard_normal((N, Ci, H, H)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci)) * np.sqrt(2.0 / Ci)).astype(np.float32)
    b = rng.uniform(-0.02, 0.02, Co).astype(np.float32)
    sets = [dict(x=CT.from_numpy(x), y=CT(), a=CT(), w=CT.from_numpy(w), b=CT.from_numpy(b), cols=CT(), ones=CT()) for _ in range(nsets)]
    g = (1, 1, 1, 1, 0, 0)

    def calls(i):
        t = sets[i]
        if fused:
            return [("convrelu_updateOutput", lambda: THNN.SpatialConvolutionMMReLU_updateOutput(t["x"], t["a"], t["w"], t["b"], t["cols"], t["ones"], *g))]
        return [("convmm_updateOutput", lambda: THNN.SpatialConvolutionMM_updateOutput(t["x"], t["y"], t["w"], t["b"], t["cols"], t["ones"], *g)),
                ("threshold_updateOutput", lambda: THNN.Threshold_updateOutput(t["y"], t["a"], 0.0, 0.0, False))]

    fl = 2.0 * Co * Ci * H * H * N
    work = ({"convrelu_updateOutput": (fl, "flops")} if fused else
            {"convmm_updateOutput": (fl, "flops"), "threshold_updateOutput": (0, "flops")})
    ns = 4

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            O.threshold_updateOutput(O.convmm_updateOutput(x[:ns], w, b, *g), 0.0, 0.0)
        return time.perf_counter() - t0, reps * ns, f"{reps} passes over {ns} images"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        ref = O.threshold_updateOutput(O.convmm_updateOutput(x[:ns], w, b, *g), 0.0, 0.0)
        np.testing.assert_allclose(t["a"].numpy()[:ns], ref, rtol=1e-5, atol=1e-4)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="mfma",
                desc=f"SpatialConvolutionMM + ReLU forward fp32 N={N} Cin={Ci} Cout={Co} {H}x{H} k1 bias, "
                     + ("fused entry point" if fused else "two separate calls"))


def wl_mbv1_block(nsets):
    """Beyond the five configurations: one MobileNet-v1 block at the shape of the metric's layer, forward then backward
    in network order - depthwise 3x3 stride 2 (128 planes, 56x56 -> 28x28) -> BatchNormalization + ReLU -> 1x1
    convolution 128 -> 128 -> BatchNormalization + ReLU, and back. All five module families of the path and the fused
    entry points in one stream: the forward and the backward pass of a layer are eight to nine launches apart, so no
    backward kernel finds its operands where the forward kernel left them."""
    from cunn_amd import CudaTensor as CT, THNN
    from oracle import oracle as O
    N, Cc, H, oH = 64, 128, 56, 28
    rng = np.random.default_rng(10)
    x = rng.standard_normal((N, Cc, H, H)).astype(np.float32)
    wd = _kaiming_uniform(rng, (1, Cc, 3, 3), 9)
    bd = rng.uniform(-1 / 3, 1 / 3, (1, Cc)).astype(np.float32)
    wp = (rng.standard_normal((Cc, Cc)) * np.sqrt(2.0 / Cc)).astype(np.float32)
    bp = rng.uniform(-0.02, 0.02, Cc).astype(np.float32)
    g1, b1 = (rng.random(Cc) + 0.5).astype(np.float32), (rng.standard_normal(Cc) * 0.1).astype(np.float32)
    g2, b2 = (rng.random(Cc) + 0.5).astype(np.float32), (rng.standard_normal(Cc) * 0.1).astype(np.float32)
    ga2 = rng.standard_normal((N, Cc, oH, oH)).astype(np.float32)      # gradient arriving from the next block
    z = lambda n=Cc: CT.from_numpy(np.zeros(n, np.float32))
    one = lambda: CT.from_numpy(np.ones(Cc, np.float32))
    sets = []
    for _ in range(nsets):
        sets.append(dict(
            x=CT.from_numpy(x), wd=CT.from_numpy(wd), bd=CT.from_numpy(bd), wp=CT.from_numpy(wp), bp=CT.from_numpy(bp),
            g1=CT.from_numpy(g1), b1=CT.from_numpy(b1), g2=CT.from_numpy(g2), b2=CT.from_numpy(b2), ga2=CT.from_numpy(ga2),
            y1=CT(), a1=CT(), y2=CT(), a2=CT(), gy2=CT.with_size(N, Cc, oH, oH), ga1=CT(), gy1=CT.with_size(N, Cc, oH, oH), gx=CT(),
            rm1=z(), rv1=one(), sm1=CT.with_size(Cc), ss1=CT.with_size(Cc), rm2=z(), rv2=one(), sm2=CT.with_size(Cc), ss2=CT.with_size(Cc),
            gg1=z(), gb1=z(), gg2=z(), gb2=z(), gwd=CT.from_numpy(np.zeros_like(wd)), gbd=CT.from_numpy(np.zeros_like(bd)),
            gwp=CT.from_numpy(np.zeros_like(wp)), gbp=z(), cd=CT(), od=CT(), cp=CT(), gcp=CT(), wcp=CT(), op=CT()))
    gd, gp = (3, 3, 2, 2, 1, 1), (1, 1, 1, 1, 0, 0)

    def calls(i):
        t = sets[i]
        return [
            ("dw_updateOutput", lambda: THNN.SpatialDepthWiseConvolution_updateOutput(t["x"], t["y1"], t["wd"], t["bd"], t["cd"], t["od"], *gd)),
            ("bnrelu1_updateOutput", lambda: THNN.BatchNormalizationReLU_updateOutput(
                t["y1"], t["a1"], t["g1"], t["b1"], t["rm1"], t["rv1"], t["sm1"], t["ss1"], True, 0.1, 1e-5)),
            ("pw_updateOutput", lambda: THNN.SpatialConvolutionMM_updateOutput(t["a1"], t["y2"], t["wp"], t["bp"], t["cp"], t["op"], *gp)),
            ("bnrelu2_updateOutput", lambda: THNN.BatchNormalizationReLU_updateOutput(
                t["y2"], t["a2"], t["g2"], t["b2"], t["rm2"], t["rv2"], t["sm2"], t["ss2"], True, 0.1, 1e-5)),
            ("bnrelu2_backward", lambda: THNN.BatchNormalizationReLU_backward(
                t["y2"], t["ga2"], t["gy2"], t["gg2"], t["gb2"], t["g2"], t["b2"], t["rm2"], t["rv2"], t["sm2"], t["ss2"], True, 1.0, 1e-5)),
            ("pw_updateGradInput", lambda: THNN.SpatialConvolutionMM_updateGradInput(t["a1"], t["gy2"], t["ga1"], t["wp"], t["gcp"], t["op"], *gp)),
            ("pw_accGradParameters", lambda: THNN.SpatialConvolutionMM_accGradParameters(
                t["a1"], t["gy2"], t["gwp"], t["gbp"], t["wcp"], t["op"], *gp, 1.0)),
            ("bnrelu1_backward", lambda: THNN.BatchNormalizationReLU_backward(
                t["y1"], t["ga1"], t["gy1"], t["gg1"], t["gb1"], t["g1"], t["b1"], t["rm1"], t["rv1"], t["sm1"], t["ss1"], True, 1.0, 1e-5)),
            ("dw_updateGradInput", lambda: THNN.SpatialDepthWiseConvolution_updateGradInput(t["x"], t["gy1"], t["gx"], t["wd"], t["cd"], t["od"], *gd)),
            ("dw_accGradParameters", lambda: THNN.SpatialDepthWiseConvolution_accGradParameters(
                t["x"], t["gy1"], t["gwd"], t["gbd"], t["cd"], t["od"], *gd, 1.0)),
        ]

    xb, yb = x.nbytes, ga2.nbytes
    # algorithmic bytes, every tensor of an entry point once; the 1x1 convolution with 128-term sums moves 2 x 25.7 MB for
    # 1.64 GFLOP (10 us of the matrix pipe): bound by memory like the rest of the block
    work = {"dw_updateOutput": (xb + yb, "bytes"), "bnrelu1_updateOutput": (2 * yb, "bytes"), "pw_updateOutput": (2 * yb, "bytes"),
            "bnrelu2_updateOutput": (2 * yb, "bytes"), "bnrelu2_backward": (3 * yb, "bytes"), "pw_updateGradInput": (2 * yb, "bytes"),
            "pw_accGradParameters": (2 * yb, "bytes"), "bnrelu1_backward": (3 * yb, "bytes"), "dw_updateGradInput": (xb + yb, "bytes"),
            "dw_accGradParameters": (xb + yb, "bytes")}

    def oracle_forward():
        y1 = O.dwconv_updateOutput(x, wd, bd, *gd)
        n1, sm1, ss1 = O.bn_updateOutput(y1, g1, b1, np.zeros(Cc, np.float32), np.ones(Cc, np.float32), True, 0.1, 1e-5)
        a1 = O.threshold_updateOutput(n1, 0.0, 0.0)
        y2 = O.convmm_updateOutput(a1, wp, bp, *gp)
        n2, sm2, ss2 = O.bn_updateOutput(y2, g2, b2, np.zeros(Cc, np.float32), np.ones(Cc, np.float32), True, 0.1, 1e-5)
        return dict(y1=y1, n1=n1, a1=a1, y2=y2, n2=n2, a2=O.threshold_updateOutput(n2, 0.0, 0.0), sm1=sm1, ss1=ss1, sm2=sm2, ss2=ss2)

    def cpu(reps):
        t0 = time.perf_counter()
        for _ in range(reps):
            f = oracle_forward()
            rm, rv = np.zeros(Cc, np.float32), np.ones(Cc, np.float32)
            gy2, _, _ = O.bn_backward(f["y2"], O.threshold_updateGradInput(f["n2"], ga2, 0.0), g2, rm, rv, f["sm2"], f["ss2"], True, 1.0,
                                      1e-5, np.zeros(Cc, np.float32), np.zeros(Cc, np.float32))
            ga1 = O.convmm_updateGradInput(f["a1"].shape, gy2, wp, *gp)
            O.convmm_accGradParameters(f["a1"], gy2, np.zeros_like(wp), np.zeros_like(bp), *gp, 1.0)
            gy1, _, _ = O.bn_backward(f["y1"], O.threshold_updateGradInput(f["n1"], ga1, 0.0), g1, rm, rv, f["sm1"], f["ss1"], True, 1.0,
                                      1e-5, np.zeros(Cc, np.float32), np.zeros(Cc, np.float32))
            O.dwconv_updateGradInput(x.shape, gy1, wd, *gd)
            O.dwconv_accGradParameters(x, gy1, np.zeros_like(wd), np.zeros_like(bd), *gd, 1.0)
        return time.perf_counter() - t0, reps * N, f"{reps} full forward + backward passes of the block ({N} images each)"

    def verify():
        t = sets[0]
        for _, fn in calls(0):
            fn()
        f = oracle_forward()
        np.testing.assert_allclose(t["a1"].numpy(), f["a1"], rtol=1e-5, atol=1e-4)
        # the second normalisation divides by the spread of a 128-term sum: deviations of the first stage pass through scaled
        np.testing.assert_allclose(t["a2"].numpy(), f["a2"], rtol=1e-4, atol=1e-4)
        for k in ("gg1", "gb1", "gg2", "gb2", "gwd", "gbd", "gwp", "gbp"):
            t[k].fill(0.0)
        for k in ("rm1", "rm2"):
            t[k].fill(0.0)
        for k in ("rv1", "rv2"):
            t[k].fill(1.0)

    return dict(calls=calls, work=work, images=N, cpu=cpu, verify=verify, bound="hbm",
                desc=f"MobileNet-v1 block fwd+bwd fp32 N={N}: depthwise 3x3 s2 {Cc}x{H}x{H} -> BN+ReLU -> 1x1 {Cc}->{Cc} at {oH}x{oH} -> BN+ReLU")


def wl_copy(nsets):
    """Calibration: plain device-to-device copy of 128 MB (2 x 128 MB of HBM traffic per launch)."""
    from cunn_amd import CudaTensor as CT
    n = 32 * 1024 * 1024
    src = np.arange(n, dtype=np.float32)
    sets = [dict(a=CT.from_numpy(src), b=CT.with_size(n)) for _ in range(nsets)]

    def calls(i):
        t = sets[i]
        return [("copy", lambda: t["b"].copy_from(t["a"]))]

    def verify():
        sets[0]["b"].copy_from(sets[0]["a"])
        assert np.array_equal(sets[0]["b"].numpy(), src)

    return dict(calls=calls, work={"copy": (2 * src.nbytes, "bytes")}, images=1, cpu=lambda reps: (1.0, 1, "n/a"),
                verify=verify, bound="hbm", desc="float4 device-to-device copy of 128 MiB")


WORKLOADS = {"copy": wl_copy, "cfg1": lambda n: wl_dw("cfg1", n), "cfg2": lambda n: wl_dw("cfg2", n), "cfg3": wl_bn, "cfg4": wl_pool,
             "dw147": lambda n: wl_dw("dw147", n), "dw14": lambda n: wl_dw("dw14", n), "pool71": lambda n: wl_pool(n, odd=True),
             "cfg5": wl_conv, "pw128": lambda n: wl_conv(n, pointwise=True), "conv1": lambda n: wl_conv(n, first=True), "dilconv": wl_dilconv, "fullconv": wl_fullconv, "relu": wl_relu,
             "bnrelu": wl_bnrelu, "bnrelu_unfused": lambda n: wl_bnrelu(n, fused=False),
             "convrelu": wl_convrelu, "convrelu_unfused": lambda n: wl_convrelu(n, fused=False), "mbv1_block": wl_mbv1_block}


PREROLL_SAMPLES = 12   # event samples per entry point collected before the timed region, whatever --warmup is
COLD_SETS = 6          # buffer sets of the cache-cold ordering
COPY_LAUNCHES = 24     # launches of the copy kernel that give the in-run streaming ceiling


def copy_ceiling(hip, stream):
    """What a plain float4 copy reaches on this part in this run: COPY_LAUNCHES launches of 128 MiB rotating through
    four buffer pairs (1 GiB, so nothing is found in the 256 MB Infinity Cache), timed by the wall clock between two
    synchronisations and, each launch on its own, by HIP events."""
    wl = wl_copy(4)
    wl["verify"]()
    fns = [wl["calls"](i)[0][1] for i in range(4)]
    nbytes = wl["work"]["copy"][0]
    for i in range(8):
        fns[i % 4]()
    ev = [(hip.event(), hip.event()) for _ in range(COPY_LAUNCHES)]
    hip.sync()
    t0 = time.perf_counter()
    for i in range(COPY_LAUNCHES):
        fns[i % 4]()
    hip.sync()
    wall = time.perf_counter() - t0
    for i, (a, b) in enumerate(ev):
        hip.record(a, stream)
        fns[i % 4]()
        hip.record(b, stream)
    hip.sync()
    med = float(np.median([hip.elapsed_ms(a, b) for a, b in ev]))
    return dict(copy_gbs=round(nbytes * COPY_LAUNCHES / wall / 1e9, 1), copy_gbs_event_median=round(nbytes / (med * 1e-3) / 1e9, 1),
                copy_bytes_per_launch=nbytes, copy_launches=COPY_LAUNCHES)


def run_workload(name, steps, warmup, hip, stream, nsets, cpu_seconds, ceiling=False, cold_sets=COLD_SETS, order="step"):
    ncold = cold_sets if nsets > 1 and name != "copy" else nsets
    if order == "cold":                  # every pass in the cache-cold ordering (for profiles of that ordering)
        ncold = max(ncold, 2)
    wl = WORKLOADS[name](max(nsets, ncold))
    wl["verify"]()                       # parity against the oracle in this very run
    names = [n for n, _ in wl["calls"](0)]
    # cache-cold ordering: the entry points of one step work on different buffer sets, `stride` sets apart, so that
    # no call finds a tensor that an earlier call of the same step (or of the step before) has touched
    stride = max(1, ncold // len(names))
    cursor = [0]                         # buffer sets keep rotating across the phases below

    def run(nsteps, bracket, cold=(order == "cold"), empty=False):
        """nsteps steps back to back; HIP events around the entry points named in `bracket`; with `empty`, one more
        event pair with nothing between them at the end of every step (what a bracket costs by itself)."""
        ev = {n: [(hip.event(), hip.event()) for _ in range(nsteps)] for n in bracket}
        if empty:
            ev[None] = [(hip.event(), hip.event()) for _ in range(nsteps)]
        hip.sync(stream)
        t0 = time.perf_counter()
        for i in range(nsteps):
            c = cursor[0]
            step = ([wl["calls"]((c + j * stride) % ncold)[j] for j in range(len(names))] if cold
                    else wl["calls"](c % nsets))
            for n, fn in step:
                if n in ev:
                    hip.record(ev[n][i][0], stream)
                    fn()
                    hip.record(ev[n][i][1], stream)
                else:
                    fn()
            if empty:
                hip.record(ev[None][i][0], stream)
                hip.record(ev[None][i][1], stream)
            cursor[0] += 1
        hip.sync(stream)
        wall = time.perf_counter() - t0
        return wall, {n: [hip.elapsed_ms(a, b) for a, b in ev[n]] for n in ev}

    def table(per_kernel):
        kern = {}
        for n in names:
            med, avg = float(np.median(per_kernel[n])), float(np.mean(per_kernel[n]))
            amount, kind = wl["work"][n]
            if kind == "bytes":
                scale, peak, unit = 1e9, HBM_PEAK_GBS, "GB/s"
            else:
                scale, peak, unit = 1e12, FP32_MFMA_PEAK_TFLOPS, "TFLOP/s"
            amount = max(amount, 1)       # entry points with no algorithmic traffic of their own (the unfused ReLU steps)
            kern[n] = dict(avg_ms=avg, median_ms=med, min_ms=float(np.min(per_kernel[n])), samples=len(per_kernel[n]),
                           achieved=amount / (avg * 1e-3) / scale, achieved_median=amount / (med * 1e-3) / scale,
                           peak=peak, unit=unit, frac=amount / (avg * 1e-3) / scale / peak,
                           frac_median=amount / (med * 1e-3) / scale / peak, algorithmic=amount, kind=kind)
        return kern

    step_work = sum(wl["work"][n][0] for n in names)
    step_scale, step_peak = (1e9, HBM_PEAK_GBS) if wl["bound"] == "hbm" else (1e12, FP32_MFMA_PEAK_TFLOPS)

    def step_frac(ms):
        return round(step_work / (ms * 1e-3) / step_scale / step_peak, 4)

    # pre-roll (untimed, reported as preroll_steps): one plain step on every buffer set, so that every
    # output / gradInput / scratch storage has its final size before anything is measured (a first call at
    # a new size allocates), then PREROLL_SAMPLES steps per entry point with HIP events around that entry
    # point alone (events around neighbouring launches would add their own few microseconds to each
    # other's bracket) - that finds the dominant kernel and times the others
    for i in range(max(nsets, ncold)):
        for _, fn in wl["calls"](i):
            fn()
    preroll = max(nsets, ncold)
    per_kernel = {}
    for n in names:
        per_kernel.update(run(PREROLL_SAMPLES, [n])[1])
        preroll += PREROLL_SAMPLES
    dominant = max(names, key=lambda n: float(np.median(per_kernel[n])))
    run(warmup, [])                      # the W warm-up steps asked for
    # the timed region: exactly `steps` steps between two synchronisations, nothing but the entry-point calls on
    # the stream - this gives `value`. Recording an event pair costs the step several microseconds (two more
    # packets for the command processor, and the kernel behind a record starts later), so the pass that brackets
    # the dominant entry point for `roofline` is a second run of the same `steps` steps right behind the first.
    wall, _ = run(steps, [])
    wall_ev, dom = run(steps, [dominant])
    per_kernel[dominant] = dom[dominant]
    _, emp = run(PREROLL_SAMPLES, [], empty=True)   # in a pass of its own: next to a real bracket it changes that bracket's reading
    kern = table(per_kernel)
    ms_per_step = wall * 1e3 / steps
    d = kern[dominant]
    traffic = load_traffic().get((name, dominant))
    roofline = dict(bound=wl["bound"], kernel=dominant, achieved=round(d["achieved"], 3), peak=d["peak"], unit=d["unit"],
                    frac=round(d["frac"], 4), traffic=traffic["bytes"] if traffic else None,
                    traffic_source=(f"profiles/{traffic['source']} at commit {traffic['commit']}" if traffic else None),
                    algorithmic_per_launch=d["algorithmic"], avg_launch_ms=round(d["avg_ms"], 5),
                    median_launch_ms=round(d["median_ms"], 5), min_launch_ms=round(d["min_ms"], 5),
                    frac_median=round(d["frac_median"], 4), samples=d["samples"],
                    step_frac=step_frac(ms_per_step), algorithmic_per_step=step_work,
                    ms_per_step_bracketed=round(wall_ev * 1e3 / steps, 5),
                    empty_bracket_ms=round(float(np.median(emp[None])), 5))
    extra = PREROLL_SAMPLES
    if ncold > len(names) and order != "cold":
        # cache-cold variant, outside the timed steps: the same entry points, each on a buffer set that nothing has
        # touched for at least `stride` - 1 whole steps (more than 1 GB of traffic at cfg2)
        run(ncold, [], cold=True)
        cold_pk = {}
        for n in names:
            cold_pk.update(run(PREROLL_SAMPLES, [n], cold=True)[1])
        cold_wall, _ = run(max(steps, 20), [], cold=True)
        ck = table(cold_pk)
        cold_ms = cold_wall * 1e3 / max(steps, 20)
        cdom = max(names, key=lambda n: ck[n]["median_ms"])
        roofline["cold"] = dict(
            order=f"entry point j of step s on buffer set (s + {stride} j) mod {ncold}", sets=ncold, kernel=cdom,
            frac=round(ck[cdom]["frac_median"], 4), ms_per_step=round(cold_ms, 5), step_frac=step_frac(cold_ms),
            entry_points={n: dict(median_ms=round(ck[n]["median_ms"], 5), min_ms=round(ck[n]["min_ms"], 5),
                                  frac=round(ck[n]["frac_median"], 4)) for n in names})
        extra += ncold + len(names) * PREROLL_SAMPLES + max(steps, 20)
    if ceiling:
        roofline.update(copy_ceiling(hip, stream))
    res = dict(workload=wl["desc"], images_per_s=wl["images"] / (ms_per_step * 1e-3), ms_per_step=ms_per_step,
               device_ms_per_step=float(sum(kern[n]["median_ms"] for n in names)), roofline=roofline, preroll_steps=preroll,
               untimed_steps_after=steps + extra,
               kernels={n: {k: (round(v, 5) if isinstance(v, float) else v) for k, v in kern[n].items()} for n in names})
    if cpu_seconds > 0 and name != "copy":
        from oracle import oracle as O
        sec, imgs, sample = wl["cpu"](1)          # calibrate
        reps = max(1, min(400, int(cpu_seconds / max(sec, 1e-3))))
        sec, imgs, sample = wl["cpu"](reps)
        res["cpu_baseline"] = dict(value=round(imgs / sec, 2), unit="images/s", cores=O.num_threads(), kind="port",
                                   sample=sample + f", {sec:.1f} s of CPU time; oracle/thnn_oracle.c with OpenMP")
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS))
    ap.add_argument("--all", action="store_true", help="also time the other four configurations")
    ap.add_argument("--sets", type=int, default=4, help="buffer sets rotated between steps (1 = cache-warm variant)")
    ap.add_argument("--cold-sets", type=int, default=COLD_SETS, help="buffer sets of the cache-cold ordering (0 = skip it)")
    ap.add_argument("--order", default="step", choices=["step", "cold"],
                    help="cold: the timed steps themselves run in the cache-cold ordering (config.order says so)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="CPU time budget of the oracle baseline (0 = skip)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(the path would shard by batch; nothing multi-GPU is built)", file=sys.stderr)
        sys.exit(2)

    import cunn_amd
    from cunn_amd.tensor import state
    lib = cunn_amd._lib.load()   # raises if libTHCUNN.so is missing: there is no fallback path
    st = state()
    stream = lib.THCState_getCurrentStream(st)
    hip = Hip()

    main_res = run_workload(args.workload, args.steps, args.warmup, hip, stream, args.sets, args.cpu_seconds, ceiling=True,
                            cold_sets=args.cold_sets, order=args.order)
    out = {
        "metric": METRIC, "value": round(main_res["images_per_s"], 1), "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(main_res["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {main_res['workload']}", "buffer_sets": args.sets if args.order == "step" else args.cold_sets,
                   "order": "every entry point of a step on the same buffer set" if args.order == "step" else "cache-cold: entry points of a step on different buffer sets",
                   "entry": "C ABI libTHCUNN.so (THNN_Cuda*) via ctypes"},
        "device_ms_per_step": round(main_res["device_ms_per_step"], 5),
        "preroll_steps": main_res["preroll_steps"],
        "untimed_steps_after": main_res["untimed_steps_after"],
        "roofline": main_res["roofline"],
        "cpu_baseline": main_res.get("cpu_baseline"),
        "kernels": main_res["kernels"],
    }
    if args.all:
        others = {}
        for name in sorted(WORKLOADS):
            if name == args.workload or name == "copy":
                continue
            r = run_workload(name, max(20, args.steps // 4), max(4, args.warmup // 2), hip, stream,
                             args.sets, min(args.cpu_seconds, 8.0))
            others[name] = dict(workload=r["workload"], images_per_s=round(r["images_per_s"], 1),
                                ms_per_step=round(r["ms_per_step"], 5), roofline=r["roofline"],
                                cpu_baseline=r.get("cpu_baseline"), kernels=r["kernels"])
        out["workloads"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()

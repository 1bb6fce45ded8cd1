"""GPU parity on shapes drawn from the ranges the reference's own tests draw from
(test.lua:1022-1033 ConvMM, :2053-2065/:2090-2103 max pooling, :2619-2632 average pooling,
:981-1015 batch normalisation), with fixed seeds so that a failure names its case.
Inputs go through makeNonContiguous-style strided tensors on every other draw, as in the
reference (test.lua:62-83). Sizes are capped so that the CPU oracle answers in seconds."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from test_gpu_parity import T, _avgpool_run, _bn_run, _conv_run, _maxpool_run, _tied_input  # noqa: E402,F401

N_DRAWS = 10


def _conv_case(seed):
    r = np.random.default_rng(1000 + seed)
    while True:
        planes = int(r.integers(1, 33))
        out = int(r.integers(1, 9)) * 8
        kW, kH = int(r.integers(3, 16)), int(r.integers(3, 16))
        dW, dH = int(r.integers(1, 4)), int(r.integers(1, 4))
        oW, oH = int(r.integers(1, 65)), int(r.integers(1, 65))
        pW, pH = int(r.integers(0, 2)), int(r.integers(0, 2))
        bs = int(r.integers(1, 5)) * 4
        W = (oW - 1) * dW + kW - 2 * pW
        H = (oH - 1) * dH + kH - 2 * pH
        flops = 2.0 * bs * out * oW * oH * planes * kW * kH
        if W >= 1 and H >= 1 and flops < 6e9 and bs * planes * H * W < 8e6:
            return (bs, planes, out, H, W, kW, kH, dW, dH, pW, pH)


@pytest.mark.parametrize("seed", range(N_DRAWS))
def test_convmm_reference_ranges(T, seed):
    case = _conv_case(seed)
    rng = np.random.default_rng(2000 + seed)
    xt = (lambda a: T.CudaTensor.noncontiguous_from_numpy(a, rng)) if seed % 2 else None
    _conv_run(T, case, bias=seed % 3 != 0, xt=xt, seed=3000 + seed)


def _pool_case(seed, avg):
    r = np.random.default_rng(4000 + seed + (500 if avg else 0))
    while True:
        planes = int(r.integers(1, 65))
        kW, kH = int(r.integers(2, 5)), int(r.integers(2, 5))
        if avg:
            dW, dH = int(r.integers(1, kW + 1)), int(r.integers(1, kH + 1))
        else:
            dW, dH = int(r.integers(1, 5)), int(r.integers(1, 5))
        oW, oH = int(r.integers(32, 129)), int(r.integers(32, 129))
        pW, pH = int(r.integers(0, kW // 2 + 1)) if kW // 2 > 0 else 0, int(r.integers(0, kH // 2 + 1)) if kH // 2 > 0 else 0
        pW, pH = min(pW, max(kW // 2 - 1, 0)) if not avg else min(pW, kW // 2), min(pH, max(kH // 2 - 1, 0)) if not avg else min(pH, kH // 2)
        ceil = bool(r.integers(0, 2))
        bs = int(r.integers(4, 11))
        W = (oW - 1) * dW + kW - 2 * pW
        H = (oH - 1) * dH + kH - 2 * pH
        if W >= kW and H >= kH and bs * planes * H * W < 1.2e7:
            return (bs, planes, H, W, kW, kH, dW, dH, pW, pH, ceil)


@pytest.mark.parametrize("seed", range(N_DRAWS))
def test_maxpool_reference_ranges(T, seed):
    case = _pool_case(seed, avg=False)
    x = _tied_input(case[:4], 5000 + seed) if seed % 2 else \
        np.random.default_rng(5000 + seed).standard_normal(case[:4]).astype(np.float32)
    rng = np.random.default_rng(5500 + seed)
    xt = T.CudaTensor.noncontiguous_from_numpy(x, rng) if seed % 3 == 0 else None
    _maxpool_run(T, case, x, xt=xt)


@pytest.mark.parametrize("seed", range(N_DRAWS))
def test_avgpool_reference_ranges(T, seed):
    case = _pool_case(seed, avg=True)
    rng = np.random.default_rng(6500 + seed)
    xt = (lambda a: T.CudaTensor.noncontiguous_from_numpy(a, rng)) if seed % 2 else None
    _avgpool_run(T, case, include_pad=bool(seed % 2), xt=xt, seed=6000 + seed)
    _avgpool_run(T, case, include_pad=not bool(seed % 2), seed=6100 + seed)


@pytest.mark.parametrize("seed", range(N_DRAWS))
def test_bn_reference_ranges(T, seed):
    r = np.random.default_rng(7000 + seed)
    shape = (int(r.integers(2, 33)), int(r.integers(1, 65)), int(r.integers(1, 65)), int(r.integers(1, 65)))
    if seed % 4 == 3:
        shape = shape[:2]  # the 1-D module
    _bn_run(T, shape, affine=bool(seed % 2), seed=7100 + seed)

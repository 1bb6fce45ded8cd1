"""Seeded random geometries for the kernels that put several small planes in one workgroup
(depthwise convolution, pooling, batch normalization with plane sizes that are not a multiple
of 4): plane sizes 1..32 on either side of every internal threshold, plane counts that leave the
last workgroup partly filled; and for the depthwise kernels that cut a larger plane of any width into
bands of rows. Same tolerances as the fixed cases."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402
from test_gpu_parity import (T, close, force_direct, _dw_run, _dw_inputs, _maxpool_run, _avgpool_run,  # noqa: E402,F401
                             _tied_input, _bn_run)


@pytest.mark.parametrize("seed", range(30))
def test_dwconv_small_random(T, seed):
    rng = np.random.default_rng(3000 + seed)
    k = int(rng.choice([3, 5]))
    s = int(rng.choice([1, 2]))
    H, W = (int(v) for v in rng.integers(1, 33, 2))
    N, C = int(rng.integers(1, 6)), int(rng.integers(1, 90))
    case = (N, C, 1, H, W, k, k, s, s, k // 2, k // 2)
    _, x, w, b = _dw_inputs(case, 3100 + seed)
    _dw_run(T, case, x, w, b if seed % 3 else None, scale=float(rng.choice([1.0, 0.25])))


# fixed shapes: network planes of odd width, a plane one row over the several-planes limit, rows so wide
# that a band is a single row, and the 5x5 window where a band's first rows lie in the border
DW_BAND_CASES = [
    (2, 3, 1, 147, 147, 3, 3, 1, 1, 1, 1),
    (1, 4, 1, 150, 150, 3, 3, 2, 2, 1, 1),
    (2, 2, 1, 75, 75, 5, 5, 2, 2, 2, 2),
    (1, 5, 1, 37, 37, 5, 5, 1, 1, 2, 2),
    (1, 3, 1, 33, 32, 3, 3, 1, 1, 1, 1),      # oW % 4 == 0 but taken as bands only if the strip kernels do not
    (1, 2, 1, 3, 2045, 3, 3, 1, 1, 1, 1),
    (1, 2, 1, 5, 1366, 5, 5, 2, 2, 2, 2),
    (1, 2, 1, 600, 3, 5, 5, 2, 2, 2, 2),
    (1, 1, 1, 1, 1025, 3, 3, 2, 2, 1, 1),
]


@pytest.mark.parametrize("case", DW_BAND_CASES, ids=lambda c: "x".join(map(str, c)))
def test_dwconv_bands(T, case):
    _, x, w, b = _dw_inputs(case, 3500)
    _dw_run(T, case, x, w, b)


@pytest.mark.parametrize("seed", range(24))
def test_dwconv_bands_random(T, seed, monkeypatch):
    rng = np.random.default_rng(3600 + seed)
    k = int(rng.choice([3, 5]))
    s = int(rng.choice([1, 2]))
    H, W = (int(v) for v in rng.integers(20, 260, 2))
    if seed % 4 == 3:  # also the widths the strip kernels would take
        monkeypatch.setenv("THCUNN_DW_SMALL", "1")
        W = W // 8 * 8 + 8
    N, C = int(rng.integers(1, 3)), int(rng.integers(1, 5))
    case = (N, C, 1, H, W, k, k, s, s, k // 2, k // 2)
    _, x, w, b = _dw_inputs(case, 3700 + seed)
    _dw_run(T, case, x, w, b if seed % 3 else None, scale=float(rng.choice([1.0, 0.5])))


@pytest.mark.parametrize("seed", range(30))
def test_pool_small_random(T, seed):
    rng = np.random.default_rng(4000 + seed)
    while True:
        kW, kH = (int(v) for v in rng.integers(1, 5, 2))
        dW, dH = (int(v) for v in rng.integers(1, 4, 2))
        pW, pH = int(rng.integers(0, kW // 2 + 1)), int(rng.integers(0, kH // 2 + 1))
        H, W = (int(v) for v in rng.integers(1, 33, 2))
        if H + 2 * pH >= kH and W + 2 * pW >= kW:
            break
    ceil = bool(rng.integers(0, 2))
    N, C = int(rng.integers(1, 5)), int(rng.integers(1, 70))
    case = (N, C, H, W, kW, kH, dW, dH, pW, pH, ceil)
    _maxpool_run(T, case, _tied_input(case[:4], 4100 + seed, q=8))
    _avgpool_run(T, case, bool(seed % 2), seed=4200 + seed)


# window geometries of the pooling kernels that work on runs of memory: (k, stride, pad)
POOL_RUN_COMBOS = [(3, 2, 1), (2, 2, 0), (3, 2, 0), (3, 1, 1)]
# network planes of odd width, planes on either side of the several-planes limit, single-row bands
POOL_RUN_PLANES = [(2, 3, 147, 147), (1, 5, 71, 71), (3, 7, 35, 35), (2, 70, 17, 17), (2, 9, 27, 27), (1, 66, 8, 8),
                   (2, 5, 28, 28), (1, 3, 45, 46), (1, 2, 3, 2045), (1, 2, 300, 3), (1, 3, 1, 1025), (2, 2, 55, 55)]


@pytest.mark.parametrize("combo", POOL_RUN_COMBOS, ids=lambda c: "k%ds%dp%d" % c)
@pytest.mark.parametrize("plane", POOL_RUN_PLANES, ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("ceil", [False, True])
def test_pool_runs(T, combo, plane, ceil):
    k, s, p = combo
    N, C, H, W = plane
    if H + 2 * p < k or W + 2 * p < k:
        pytest.skip("window larger than the padded plane")
    case = (N, C, H, W, k, k, s, s, p, p, ceil)
    _maxpool_run(T, case, _tied_input(case[:4], 4500, q=8))
    _avgpool_run(T, case, True, seed=4501)
    _avgpool_run(T, case, False, seed=4502)


@pytest.mark.parametrize("seed", range(24))
def test_pool_runs_random(T, seed):
    rng = np.random.default_rng(4600 + seed)
    k, s, p = POOL_RUN_COMBOS[seed % 4]
    H, W = (int(v) for v in rng.integers(max(1, k - 2 * p), 200, 2))
    N, C = int(rng.integers(1, 4)), int(rng.integers(1, 40))
    case = (N, C, H, W, k, k, s, s, p, p, bool(rng.integers(0, 2)))
    _maxpool_run(T, case, _tied_input(case[:4], 4700 + seed, q=8))
    _avgpool_run(T, case, bool(seed % 2), seed=4800 + seed)


# widths that are multiples of 4: the strip kernels and the run kernels both apply, the library picks by size
POOL_BOTH_PLANES = [(2, 9, 27, 27), (1, 5, 71, 71), (2, 70, 17, 17), (2, 6, 56, 56), (1, 4, 112, 112), (2, 8, 16, 16),
                    (1, 3, 32, 64), (1, 2, 8, 8)]


@pytest.mark.parametrize("combo", POOL_RUN_COMBOS, ids=lambda c: "k%ds%dp%d" % c)
@pytest.mark.parametrize("switch", ["0", "1"])
def test_pool_runs_switch(T, combo, switch):
    """THCUNN_POOL_RUNS=0: never the run kernels (strip kernels, small-plane kernels, tiled kernels as before);
    1: the run kernels wherever their window geometry matches."""
    k, s, p = combo
    with force_direct("THCUNN_POOL_RUNS", switch):
        for plane in POOL_BOTH_PLANES:
            for ceil in (False, True):
                case = plane + (k, k, s, s, p, p, ceil)
                _maxpool_run(T, case, _tied_input(case[:4], 4900, q=8))
                _avgpool_run(T, case, not ceil, seed=4901)


@pytest.mark.parametrize("seed", range(16))
def test_batchnorm_small_random(T, seed):
    rng = np.random.default_rng(5000 + seed)
    H, W = (int(v) for v in rng.integers(1, 12, 2))
    N, C = int(rng.integers(1, 80)), int(rng.integers(96, 140))
    _bn_run(T, (N, C, H, W), bool(seed % 2), seed=5100 + seed)


# plane sizes that are not multiples of 4 beyond the 256-lane resident kernels: 1024-lane resident kernels
# (channels of up to 32768 elements, >= 96 channels) and the chunked kernels with 16-byte accesses around
# unaligned plane starts (whole planes per chunk, and planes cut into segments)
BN_ODD_SHAPES = [(32, 100, 17, 17), (64, 96, 13, 13), (30, 97, 27, 27), (32, 96, 31, 31), (17, 101, 35, 35),
                 (4, 8, 35, 35), (3, 5, 147, 147), (2, 3, 99, 101), (5, 7, 3, 3), (6, 4, 1, 9), (2, 130, 75, 75)]


@pytest.mark.parametrize("shape", BN_ODD_SHAPES, ids=lambda c: "x".join(map(str, c)))
def test_batchnorm_odd_planes(T, shape):
    _bn_run(T, shape, True, seed=5200)


@pytest.mark.parametrize("shape", BN_ODD_SHAPES[:4] + BN_ODD_SHAPES[6:7], ids=lambda c: "x".join(map(str, c)))
def test_batchnorm_odd_planes_chunked(T, shape):
    with force_direct("THCUNN_BN_FORCE_CHUNKED", "1"):
        _bn_run(T, shape, False, seed=5201)


def _at_offset(T, a, off):
    """A contiguous tensor whose first element sits `off` floats behind a 16-byte boundary of its storage."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    big = T.CudaTensor.with_size(a.size + 8)
    big.fill(float("nan"))
    strides = [1] * a.ndim
    for d in range(a.ndim - 2, -1, -1):
        strides[d] = strides[d + 1] * a.shape[d + 1]
    v = big.view(off, a.shape, strides)
    v.copy_(a)
    return v


@pytest.mark.parametrize("off", [1, 2, 3])
def test_run_kernels_decline_unaligned_tensors(T, off):
    """The run-of-memory kernels fetch from the 16-byte boundary below a run and so need 16-byte aligned
    tensors; an input that starts elsewhere in its storage takes the other kernels, with the same results."""
    THNN, CT, LT = T.THNN, T.CudaTensor, T.CudaLongTensor
    rng = np.random.default_rng(6000 + off)
    # depthwise convolution, small planes
    case = (2, 9, 1, 14, 14, 3, 3, 1, 1, 1, 1)
    _, x, w, b = _dw_inputs(case, 6100 + off)
    _dw_run(T, case, x, w, b, xt=_at_offset(T, x, off))
    # pooling, odd width
    x = _tied_input((2, 5, 27, 27), 6200 + off, q=8)
    _maxpool_run(T, (2, 5, 27, 27, 3, 3, 2, 2, 0, 0, False), x, xt=_at_offset(T, x, off))
    tx, out = _at_offset(T, x, off), CT()
    THNN.SpatialAveragePooling_updateOutput(tx, out, 3, 3, 2, 2, 0, 0, False, True)
    close(out.numpy(), O.avgpool_updateOutput(x, 3, 3, 2, 2, 0, 0, False, True))
    # batch normalization, plane size not a multiple of 4
    shape = (6, 5, 9, 9)
    x = rng.standard_normal(shape).astype(np.float32)
    C = shape[1]
    v = lambda a: CT.from_numpy(np.asarray(a, np.float32))
    rm, rv, sm, ss = v(np.zeros(C)), v(np.ones(C)), v(np.zeros(C)), v(np.zeros(C))
    out = CT()
    THNN.BatchNormalization_updateOutput(_at_offset(T, x, off), out, None, None, rm, rv, sm, ss, True, 0.1, 1e-5)
    mean = x.mean(axis=(0, 2, 3), keepdims=True, dtype=np.float64)
    var = x.var(axis=(0, 2, 3), keepdims=True, dtype=np.float64)
    close(out.numpy(), ((x - mean) / np.sqrt(var + 1e-5)).astype(np.float32))

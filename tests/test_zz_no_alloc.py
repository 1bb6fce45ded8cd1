"""SpatialDepthWiseConvolution_accGradParameters_noAlloc (no counterpart in the reference: the variant
for callers that cannot allocate device memory) against the regular entry point, through the C ABI.

Both run the same kernels in the same order, so the results must be bit-identical; the regular entry
point is itself checked against the CPU oracle here at the weight-gradient tolerance (1e-3 relative).
Calls on one GPU share one scratch array that keeps the last call's contents, so every case is run as
two calls in a row, the second on a smaller input.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402

WG_RTOL, WG_ATOL = 1e-3, 1e-4


@pytest.fixture(scope="module")
def T():
    import cunn_amd
    return cunn_amd


def _both(T, case, seed, scale, bias=True):
    """(gradWeight, gradBias) of the regular and of the no-allocation entry point, plus the oracle's."""
    N, C, M, H, W, k, s, p = case
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(seed)
    oH, oW = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    gy = rng.standard_normal((N, C * M, oH, oW)).astype(np.float32)
    gw0 = rng.standard_normal((M, C, k, k)).astype(np.float32)      # accumulate into non-zero gradients
    gb0 = rng.standard_normal((M, C)).astype(np.float32)
    tx, tgy = CT.from_numpy(x), CT.from_numpy(gy)
    g = (k, k, s, s, p, p)
    gw_a, gb_a = CT.from_numpy(gw0), (CT.from_numpy(gb0) if bias else None)
    THNN.SpatialDepthWiseConvolution_accGradParameters(tx, tgy, gw_a, gb_a, CT(), CT(), *g, scale)
    gw_b, gb_b = CT.from_numpy(gw0), (CT.from_numpy(gb0) if bias else None)
    THNN.SpatialDepthWiseConvolution_accGradParameters_noAlloc(tx, tgy, gw_b, gb_b, *g, scale)
    rgw, rgb = O.dwconv_accGradParameters(x, gy, gw0.copy(), gb0.copy(), *g, scale)
    return ((gw_a.numpy(), gb_a.numpy() if bias else None), (gw_b.numpy(), gb_b.numpy() if bias else None), (rgw, rgb))


# (first call, second call on a smaller input); N, C, M, H, W, k, stride, pad
PAIRS = [
    ((8, 32, 1, 56, 56, 3, 2, 1), (2, 8, 1, 28, 28, 3, 2, 1)),       # strip kernels, then several planes per workgroup
    ((4, 16, 1, 112, 112, 3, 1, 1), (3, 5, 1, 20, 24, 3, 1, 1)),     # bands of rows, then a small odd channel count
    ((2, 6, 2, 30, 34, 5, 1, 2), (1, 3, 2, 12, 16, 5, 1, 2)),        # depth multiplier 2 (generic band kernels)
    ((2, 4, 1, 37, 37, 3, 1, 1), (1, 2, 1, 7, 7, 3, 1, 1)),          # widths that are not multiples of 4
    ((1, 3, 2, 17, 19, 3, 2, 0), (1, 2, 1, 9, 9, 3, 2, 0)),          # no padding: neither fast family
]


@pytest.mark.parametrize("first,second", PAIRS)
@pytest.mark.parametrize("bias", [True, False])
def test_no_alloc_matches_regular_entry_point_twice_in_a_row(T, first, second, bias):
    for i, case in enumerate((first, second)):
        print("case", case, "bias", bias, flush=True)
        (gw_a, gb_a), (gw_b, gb_b), (rgw, rgb) = _both(T, case, seed=11 + i, scale=0.5 + i, bias=bias)
        assert np.array_equal(gw_a, gw_b)
        np.testing.assert_allclose(gw_a, rgw, rtol=WG_RTOL, atol=WG_ATOL)
        if bias:
            assert np.array_equal(gb_a, gb_b)
            np.testing.assert_allclose(gb_a, rgb, rtol=WG_RTOL, atol=WG_ATOL)


def test_no_alloc_headline_shape_then_smaller(T):
    """The shape the metric is quoted on (327 KB of partial sums), then a quarter of it."""
    for i, case in enumerate(((64, 128, 1, 56, 56, 3, 2, 1), (16, 128, 1, 56, 56, 3, 2, 1))):
        print("case", case, flush=True)
        (gw_a, gb_a), (gw_b, gb_b), (rgw, rgb) = _both(T, case, seed=21 + i, scale=1.0)
        assert np.array_equal(gw_a, gw_b) and np.array_equal(gb_a, gb_b)
        np.testing.assert_allclose(gw_a, rgw, rtol=WG_RTOL, atol=2e-3)
        np.testing.assert_allclose(gb_a, rgb, rtol=WG_RTOL, atol=2e-3)


def test_no_alloc_refuses_what_would_allocate(T):
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(3)
    g = (3, 3, 1, 1, 1, 1)
    x = rng.standard_normal((2, 4, 16, 16)).astype(np.float32)
    gy = rng.standard_normal((2, 4, 16, 16)).astype(np.float32)
    gw, gb = CT.from_numpy(np.zeros((1, 4, 3, 3), np.float32)), CT.from_numpy(np.zeros((1, 4), np.float32))
    # a strided input would have to be packed into a temporary
    xs = CT.noncontiguous_from_numpy(x, rng)
    if not xs.is_contiguous():
        with pytest.raises(T.THError, match="contiguous"):
            THNN.SpatialDepthWiseConvolution_accGradParameters_noAlloc(xs, CT.from_numpy(gy), gw, gb, *g, 1.0)
    # a 2-D gradWeight would be reshaped in place
    gw2 = CT.from_numpy(np.zeros((1, 36), np.float32))
    with pytest.raises(T.THError, match="4D gradWeight"):
        THNN.SpatialDepthWiseConvolution_accGradParameters_noAlloc(CT.from_numpy(x), CT.from_numpy(gy), gw2, gb, *g, 1.0)
    # more partial sums than the fixed scratch holds: 2048 channels x 10 taps x 64 images = 1.3 M floats
    N, Cc = 64, 2048
    xb = CT.with_size(N, Cc, 8, 8).fill(0.0)
    gyb = CT.with_size(N, Cc, 8, 8).fill(0.0)
    gwb, gbb = CT.from_numpy(np.zeros((1, Cc, 3, 3), np.float32)), CT.from_numpy(np.zeros((1, Cc), np.float32))
    with pytest.raises(T.THError, match="fixed scratch holds"):
        THNN.SpatialDepthWiseConvolution_accGradParameters_noAlloc(xb, gyb, gwb, gbb, *g, 1.0)
    # and the gradients were left alone
    assert not gwb.numpy().any() and not gbb.numpy().any()
    # the regular entry point still takes all three
    THNN.SpatialDepthWiseConvolution_accGradParameters(xs, CT.from_numpy(gy), gw, gb, CT(), CT(), *g, 1.0)
    rgw, rgb = O.dwconv_accGradParameters(x, gy, np.zeros((1, 4, 3, 3), np.float32), np.zeros((1, 4), np.float32), *g, 1.0)
    np.testing.assert_allclose(gw.numpy(), rgw, rtol=WG_RTOL, atol=WG_ATOL)


def test_no_alloc_two_host_threads_never_share_the_scratch_silently(T):
    """All calls on a GPU share one scratch array. Two host threads that are inside the entry point at the same time
    are told so (TH error, nothing launched) instead of folding each other's partial sums; a call that does go
    through gives the regular entry point's bits. Both threads issue on the device's default stream, so the launches
    of calls that did not overlap on the host do not overlap on the GPU either."""
    import threading

    from cunn_amd import tensor as TT
    lib = T._lib.load()
    CT, THNN = T.CudaTensor, T.THNN
    g = (3, 3, 2, 2, 1, 1)
    work = []
    for seed, (N, C) in enumerate(((8, 32), (6, 24))):
        rng = np.random.default_rng(40 + seed)
        x, gy = rng.standard_normal((N, C, 56, 56)).astype(np.float32), rng.standard_normal((N, C, 28, 28)).astype(np.float32)
        gw0, gb0 = rng.standard_normal((1, C, 3, 3)).astype(np.float32), rng.standard_normal((1, C)).astype(np.float32)
        tx, tgy = CT.from_numpy(x), CT.from_numpy(gy)
        ref_w, ref_b = CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.SpatialDepthWiseConvolution_accGradParameters(tx, tgy, ref_w, ref_b, CT(), CT(), *g, 1.0)
        work.append(dict(x=tx, gy=tgy, gw0=gw0, gb0=gb0, ref_w=ref_w.numpy(), ref_b=ref_b.numpy(),
                         gw=CT.from_numpy(gw0), gb=CT.from_numpy(gb0), done=0, refused=0, wrong=0))
    TT.synchronize()
    del TT._pending[:]
    ROUNDS = 200

    import ctypes as C

    def put(st, t, a):      # the harness's own copy helpers raise on any pending TH error, also the other thread's
        lib.THCudaTensor_copyFromHost(st, t.handle, a.ctypes.data_as(C.c_void_p))

    def get(st, t, like):
        out = np.empty_like(like)
        lib.THCudaTensor_copyToHost(st, t.handle, out.ctypes.data_as(C.c_void_p))
        return out

    def run(w):
        st = lib.THCState_alloc()
        for _ in range(ROUNDS):
            put(st, w["gw"], w["gw0"]), put(st, w["gb"], w["gb0"])
            lib.THNN_CudaSpatialDepthWiseConvolution_accGradParameters_noAlloc(
                st, w["x"].handle, w["gy"].handle, w["gw"].handle, w["gb"].handle, *g, 1.0)
            lib.THCState_synchronize(st)
            gw, gb = get(st, w["gw"], w["gw0"]), get(st, w["gb"], w["gb0"])
            if np.array_equal(gw, w["ref_w"]) and np.array_equal(gb, w["ref_b"]):
                w["done"] += 1
            elif np.array_equal(gw, w["gw0"]) and np.array_equal(gb, w["gb0"]):
                w["refused"] += 1
            else:
                w["wrong"] += 1
        lib.THCState_free(st)

    threads = [threading.Thread(target=run, args=(w,)) for w in work]
    [t.start() for t in threads]
    [t.join() for t in threads]
    errors = list(TT._pending)
    del TT._pending[:]
    print("done", [w["done"] for w in work], "refused", [w["refused"] for w in work], flush=True)
    assert all(w["wrong"] == 0 for w in work)
    assert all(w["done"] > 0 for w in work)
    assert len(errors) == sum(w["refused"] for w in work) and all("must not overlap" in e for e in errors)

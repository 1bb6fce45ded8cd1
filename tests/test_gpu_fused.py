"""BatchNormalization + Threshold(0, 0) in one pass (include/THCUNN_fused.h; no counterpart in the reference's
C ABI) against the oracle's composition of the two modules it fuses:

    forward   threshold_updateOutput(bn_updateOutput(x), 0, 0)
    backward  bn_backward(x, threshold_updateGradInput(y, gradOutput, 0))

and, bit for bit, against this library's own two-call sequence (the fused kernels use the same arithmetic).
Where the normalised value is within rounding of 0 its sign - hence the ReLU mask - is not determined by the
mathematics (fp32 here, double accumulators in the oracle); gradOutput is set to 0 on those few elements, so
the mask there cannot reach any result. Tolerances: 1e-5 relative / 1e-4 absolute for outputs and gradInput,
1e-3 relative for the statistics and the weight / bias gradients.
"""
import numpy as np
import pytest

import cunn_amd

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402

SHAPES = [
    (8, 16, 28, 28),      # chunked two-pass kernels (few channels)
    (64, 100, 28, 28),    # channel-resident kernels, x kept in registers
    (64, 128, 28, 28),    # channel-resident, 13 float4 per lane: x parked in LDS / re-read
    (40, 96, 20, 20),
    (16, 130, 7, 7),      # small channels, plane size not a multiple of 4
    (160, 97, 7, 7),
    (2, 5, 33),           # element by element
    (32, 64),             # 2-D input
    (2, 2, 150, 120),     # planes cut into segments
    (3, 7, 35, 35),       # 16-byte accesses around unaligned plane starts
]


def _run(shape, affine, train, seed, forced_chunked=False):
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(seed)
    Cc = shape[1]
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float32)
    g = (rng.random(Cc) + 0.25).astype(np.float32) if affine else None
    b = rng.standard_normal(Cc).astype(np.float32) if affine else None
    rm0 = rng.standard_normal(Cc).astype(np.float32) * 0.3 + 0.5
    rv0 = (rng.random(Cc) * 2 + 3).astype(np.float32)
    eps, mom, scale = 1e-5, 0.1, 0.5
    v = lambda a: None if a is None else CT.from_numpy(a)
    tx, tg, tb = CT.from_numpy(x), v(g), v(b)

    def forward(fn):
        rm, rv, sm, ss, out = CT.from_numpy(rm0), CT.from_numpy(rv0), CT.with_size(Cc), CT.with_size(Cc), CT()
        fn(tx, out, tg, tb, rm, rv, sm, ss, train, mom, eps)
        return out, rm, rv, sm, ss

    if forced_chunked:
        cunn_amd.set_switch("THCUNN_BN_FORCE_CHUNKED", "1")
    try:
        fused, frm, frv, fsm, fss = forward(THNN.BatchNormalizationReLU_updateOutput)
        plain, prm, prv, psm, pss = forward(THNN.BatchNormalization_updateOutput)
        relu = CT()
        THNN.Threshold_updateOutput(plain, relu, 0.0, 0.0, False)
        # oracle composition
        orm, orv = rm0.copy(), rv0.copy()
        y_pre, osm, oss = O.bn_updateOutput(x, g, b, orm, orv, train, mom, eps)
        y_ref = O.threshold_updateOutput(y_pre, 0.0, 0.0)
        fo = fused.numpy()
        assert fo.shape == tuple(shape)
        np.testing.assert_allclose(fo, y_ref, rtol=1e-5, atol=1e-4)
        assert np.array_equal(fo, relu.numpy())                      # same arithmetic as the two calls
        for a, r in ((frm, prm), (frv, prv)) + (((fsm, psm), (fss, pss)) if train else ()):
            assert np.array_equal(a.numpy(), r.numpy())
        if train:
            np.testing.assert_allclose(fsm.numpy(), osm, rtol=1e-3, atol=1e-5)
            np.testing.assert_allclose(fss.numpy(), oss, rtol=1e-3, atol=1e-6)

        # backward; gradOutput vanishes where the sign of the normalised value is within rounding of undecided
        gy = rng.standard_normal(shape).astype(np.float32)
        gy[np.abs(y_pre) < 1e-4] = 0.0
        tgy = CT.from_numpy(gy)
        gw0, gb0 = rng.standard_normal(Cc).astype(np.float32), rng.standard_normal(Cc).astype(np.float32)
        gi, tgw, tgb = CT.with_size(*shape), CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.BatchNormalizationReLU_backward(tx, tgy, gi, tgw, tgb, tg, tb, frm, frv, fsm, fss, train, scale, eps)
        masked = O.threshold_updateGradInput(y_pre, gy, 0.0)
        rgi, rgw, rgb = O.bn_backward(x, masked, g, orm, orv, osm, oss, train, scale, eps, gw0.copy(), gb0.copy())
        np.testing.assert_allclose(gi.numpy(), rgi, rtol=1e-5, atol=1e-4)
        np.testing.assert_allclose(tgw.numpy(), rgw, rtol=1e-3, atol=1e-3)
        np.testing.assert_allclose(tgb.numpy(), rgb, rtol=1e-3, atol=1e-3)
        # the library's own two calls: Threshold backward, then BatchNormalization backward
        tmasked = CT()
        THNN.Threshold_updateGradInput(relu, tgy, tmasked, 0.0, 0.0, False)
        gi2, tgw2, tgb2 = CT.with_size(*shape), CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.BatchNormalization_backward(tx, tmasked, gi2, tgw2, tgb2, tg, prm, prv, psm, pss, train, scale, eps)
        assert np.array_equal(gi.numpy(), gi2.numpy())
        assert np.array_equal(tgw.numpy(), tgw2.numpy()) and np.array_equal(tgb.numpy(), tgb2.numpy())
        # split order (gradInput alone, then the parameter gradients alone), as the nn module may call it
        gi3 = CT.with_size(*shape)
        THNN.BatchNormalizationReLU_backward(tx, tgy, gi3, None, None, tg, tb, frm, frv, fsm, fss, train, scale, eps)
        tgw3, tgb3 = CT.from_numpy(gw0), CT.from_numpy(gb0)
        THNN.BatchNormalizationReLU_backward(tx, tgy, None, tgw3, tgb3, tg, tb, frm, frv, fsm, fss, train, scale, eps)
        assert np.array_equal(gi.numpy(), gi3.numpy())
        assert np.array_equal(tgw.numpy(), tgw3.numpy()) and np.array_equal(tgb.numpy(), tgb3.numpy())
    finally:
        if forced_chunked:
            cunn_amd.set_switch("THCUNN_BN_FORCE_CHUNKED", None)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("affine", [True, False])
@pytest.mark.parametrize("train", [True, False])
def test_batchnorm_relu(shape, affine, train):
    print("shape", shape, "affine", affine, "train", train, flush=True)
    _run(shape, affine, train, seed=60)


@pytest.mark.parametrize("shape", [(64, 100, 28, 28), (16, 130, 7, 7)])
def test_batchnorm_relu_chunked_kernels_on_resident_shapes(shape):
    _run(shape, True, True, seed=61, forced_chunked=True)


def test_batchnorm_relu_cfg3_shape():
    """The BatchNormalization configuration of the benchmark (64 x 256 x 28 x 28), fused."""
    _run((64, 256, 28, 28), True, True, seed=2)


def test_batchnorm_relu_strided_input():
    THNN, CT = cunn_amd.THNN, cunn_amd.CudaTensor
    rng = np.random.default_rng(62)
    shape, Cc = (4, 6, 9, 10), 6
    x = rng.standard_normal(shape).astype(np.float32)
    g, b = rng.random(Cc).astype(np.float32) + 0.5, rng.standard_normal(Cc).astype(np.float32)
    rm, rv = CT.from_numpy(np.zeros(Cc, np.float32)), CT.from_numpy(np.ones(Cc, np.float32))
    sm, ss, out = CT.with_size(Cc), CT.with_size(Cc), CT()
    THNN.BatchNormalizationReLU_updateOutput(CT.noncontiguous_from_numpy(x, rng), out, CT.from_numpy(g), CT.from_numpy(b),
                                             rm, rv, sm, ss, True, 0.1, 1e-5)
    y_pre, _, _ = O.bn_updateOutput(x, g, b, np.zeros(Cc, np.float32), np.ones(Cc, np.float32), True, 0.1, 1e-5)
    np.testing.assert_allclose(out.numpy(), O.threshold_updateOutput(y_pre, 0.0, 0.0), rtol=1e-5, atol=1e-4)

"""GPU parity of Threshold (bit-exact: the op only selects values) through the C ABI: odd sizes
(scalar tail), non-contiguous inputs and outputs, the in-place variants (the result tensor becomes
a view of the overwritten one, generic/Threshold.cu:18-25, 50-56), NaN / threshold-equal inputs,
the nElement check."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402
from test_gpu_parity import T  # noqa: E402,F401


@pytest.mark.parametrize("shape", [(4, 8, 14, 14), (3, 5, 7), (1031,), (2, 3, 5, 9, 4), (1,)])
@pytest.mark.parametrize("thr,val", [(0.0, 0.0), (0.3, -2.0)])
def test_threshold(T, shape, thr, val):
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(100)
    x = rng.standard_normal(shape).astype(np.float32)
    x.flat[0] = thr
    if x.size > 2:
        x.flat[1] = np.nan
    gy = rng.standard_normal(shape).astype(np.float32)
    out, gi = CT(), CT()
    THNN.Threshold_updateOutput(CT.from_numpy(x), out, thr, val, False)
    assert out.size() == tuple(shape)
    assert np.array_equal(out.numpy(), O.threshold_updateOutput(x, thr, val), equal_nan=True)
    THNN.Threshold_updateGradInput(CT.from_numpy(x), CT.from_numpy(gy), gi, thr, val, False)
    assert np.array_equal(gi.numpy(), O.threshold_updateGradInput(x, gy, thr))


def test_threshold_noncontiguous_and_inplace(T):
    THNN, CT = T.THNN, T.CudaTensor
    rng = np.random.default_rng(101)
    x = rng.standard_normal((3, 6, 10, 12)).astype(np.float32)
    gy = rng.standard_normal(x.shape).astype(np.float32)
    tx = CT.noncontiguous_from_numpy(x, rng)
    tgy = CT.noncontiguous_from_numpy(gy, rng)
    assert not tx.is_contiguous()
    out, gi = CT(), CT()
    THNN.Threshold_updateOutput(tx, out, 0.1, 0.5, False)
    assert np.array_equal(out.numpy(), O.threshold_updateOutput(x, 0.1, 0.5))
    THNN.Threshold_updateGradInput(tx, tgy, gi, 0.1, 0.5, False)
    assert np.array_equal(gi.numpy(), O.threshold_updateGradInput(x, gy, 0.1))
    # in place: through the strides of a non-contiguous tensor and on a contiguous one
    for mk in (lambda a: CT.noncontiguous_from_numpy(a, rng), CT.from_numpy):
        ti, tg = mk(x), mk(gy)
        o2, g2 = CT(), CT()
        THNN.Threshold_updateGradInput(ti, tg, g2, 0.1, 0.5, True)      # gradOutput is overwritten, input still intact
        assert np.array_equal(tg.numpy(), O.threshold_updateGradInput(x, gy, 0.1))
        assert np.array_equal(g2.numpy(), tg.numpy()) and g2.size() == tg.size()
        THNN.Threshold_updateOutput(ti, o2, 0.1, 0.5, True)
        assert np.array_equal(ti.numpy(), O.threshold_updateOutput(x, 0.1, 0.5))
        assert np.array_equal(o2.numpy(), ti.numpy()) and o2.size() == ti.size()
        if ti.is_contiguous():
            ti.fill(7.0)                                                # the result is a view: it follows its source
            assert np.all(o2.numpy() == 7.0)


def test_threshold_errors(T):
    THNN, CT = T.THNN, T.CudaTensor
    x = CT.from_numpy(np.zeros((2, 3), np.float32))
    g = CT.from_numpy(np.zeros((2, 4), np.float32))
    with pytest.raises(T.THError, match="have different number of elements"):
        THNN.Threshold_updateGradInput(x, g, CT(), 0.0, 0.0, False)

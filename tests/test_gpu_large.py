"""Sizes at and beyond the 32-bit limits of the launch helpers (lib/THCUNN/common.h:5-83 counts elements in
`int`): tensors of more than 2^31 bytes run through the C ABI against the oracle, and extents that the
kernels' 32-bit plane arithmetic cannot hold are refused with a TH error before anything is launched."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from oracle import oracle as O  # noqa: E402


@pytest.fixture(scope="module")
def T():
    import cunn_amd
    return cunn_amd


# 40 x 128 planes of 336 x 336 floats: 2.31e9 bytes, past 2^31 = 2.147e9
BIG = (40, 128, 336, 336)


def test_depthwise_forward_beyond_2_gib(T):
    CT, THNN = T.CudaTensor, T.THNN
    assert np.prod(BIG) * 4 > 2 ** 31
    rng = np.random.default_rng(90)
    x = rng.random(BIG, dtype=np.float32) - 0.5
    C = BIG[1]
    w = rng.uniform(-0.8, 0.8, (1, C, 3, 3)).astype(np.float32)
    b = rng.uniform(-0.3, 0.3, (1, C)).astype(np.float32)
    y = CT()
    print("depthwise forward", BIG, flush=True)
    THNN.SpatialDepthWiseConvolution_updateOutput(CT.from_numpy(x), y, CT.from_numpy(w), CT.from_numpy(b), CT(), CT(),
                                                  3, 3, 1, 1, 1, 1)
    yv = y.numpy()
    assert yv.shape == BIG
    np.testing.assert_allclose(yv, O.dwconv_updateOutput(x, w, b, 3, 3, 1, 1, 1, 1), rtol=1e-5, atol=1e-4)


def test_maxpool_beyond_2_gib(T):
    CT, LT, THNN = T.CudaTensor, T.CudaLongTensor, T.THNN
    rng = np.random.default_rng(91)
    x = np.round((rng.random(BIG, dtype=np.float32) - 0.5) * 128) / 64          # ties
    M = (3, 3, 2, 2, 1, 1, False)
    tx, y, idx = CT.from_numpy(x), CT(), LT()
    print("max pooling forward", BIG, flush=True)
    THNN.SpatialMaxPooling_updateOutput(tx, y, idx, *M)
    yv, iv = y.numpy(), idx.numpy()
    ry, ridx = O.maxpool_updateOutput(x, *M)
    assert np.array_equal(yv, ry) and np.array_equal(iv, ridx)                    # bit-exact, values and argmax
    # index round trip over the whole tensor: the argmax position holds the maximum
    N, C, H, W = BIG
    flat = x.reshape(N * C, H * W)
    assert np.array_equal(np.take_along_axis(flat, iv.reshape(N * C, -1) - 1, axis=1), yv.reshape(N * C, -1))
    del ry, flat
    gy = rng.random(yv.shape, dtype=np.float32) - 0.5
    gx = CT()
    print("max pooling backward", BIG, flush=True)
    THNN.SpatialMaxPooling_updateGradInput(tx, CT.from_numpy(gy), gx, idx, *M)
    gxv = gx.numpy()
    assert gxv.shape == BIG
    np.testing.assert_allclose(gxv, O.maxpool_updateGradInput(BIG, gy, ridx, *M), rtol=1e-5, atol=1e-4)


def _fake(T, size):
    """A tensor that claims `size` (contiguous strides) over a 16-float storage: for calls that must be
    refused before any kernel reads it."""
    strides, z = [], 1
    for s in reversed(size):
        strides.append(z)
        z *= s
    return T.CudaTensor.with_size(16).view(0, size, list(reversed(strides)))


def test_extents_beyond_the_plane_arithmetic_are_refused(T):
    CT, LT, THNN = T.CudaTensor, T.CudaLongTensor, T.THNN
    # pooling: a plane of 2^31 elements
    with pytest.raises(T.THError, match="2\\^31 or more elements"):
        THNN.SpatialMaxPooling_updateOutput(_fake(T, (1, 1, 65536, 32768)), CT(), LT(), 3, 3, 2, 2, 1, 1, False)
    with pytest.raises(T.THError, match="2\\^31 or more elements"):
        THNN.SpatialAveragePooling_updateOutput(_fake(T, (1, 1, 65536, 32768)), CT(), 2, 2, 2, 2, 0, 0, False, True)
    # batch normalization: 2^31 elements per (image, channel)
    C = 2
    v = lambda a: CT.from_numpy(np.asarray(a, np.float32))
    with pytest.raises(T.THError, match="2\\^31 or more elements"):
        THNN.BatchNormalization_updateOutput(_fake(T, (2, C, 2 ** 31)), CT(), None, None, v(np.zeros(C)), v(np.ones(C)),
                                             v(np.zeros(C)), v(np.zeros(C)), True, 0.1, 1e-5)
    # convolution: an image of 2^32 elements
    w, b = v(np.zeros((8, 36))), v(np.zeros(8))
    with pytest.raises(T.THError, match="image too large"):
        THNN.SpatialConvolutionMM_updateOutput(_fake(T, (1, 4, 32768, 32768)), CT(), w, b, CT(), CT(), 3, 3, 1, 1, 1, 1)

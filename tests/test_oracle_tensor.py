"""Pins of the oracle's transform and reduce-sum functions (CPU only).

The reference's own test (legacy/tests/tensor/test_tensor_mpi_cuda_algorithms.cu)
fills a tensor with the global offset of each element, doubles it with Transform,
copies it, and reduces it: each reduced cell must equal the plain sum, and the
nested reduction to one cell (size - 1) * size / 2 (:100-300).  Those closed forms,
brute-force loops and the batch-norm statistics closed form are used here."""
import numpy as np
import pytest

import oracle


def _offsets(shape):
    return np.arange(int(np.prod(shape)), dtype=np.float64).reshape(shape)


def test_transform_times_two_copy_and_affine_closed_forms():
    shape = (3, 4, 5, 6)
    halo = np.full((3, 4, 7, 10), np.nan, np.float32)   # halos of 1 and 2 around the two inner axes
    interior = halo[:, :, 1:6, 2:8]
    interior[...] = _offsets(shape)
    oracle.tensor_transform(oracle.TRANSFORM_SCALE, [interior], [2.0])
    assert np.array_equal(interior, 2 * _offsets(shape))           # times2_functor, :126-146
    assert np.isnan(halo[:, :, 0, :]).all() and np.isnan(halo[:, :, :, :2]).all()   # halo untouched
    other = np.zeros(shape, np.float32)
    oracle.tensor_transform(oracle.TRANSFORM_COPY, [interior, other])
    assert np.array_equal(other, 2 * _offsets(shape))              # copy_functor, :147-159
    oracle.tensor_transform(oracle.TRANSFORM_SCALE_BIAS, [interior, other], [0.5, 3.0])
    assert np.array_equal(other, _offsets(shape) + 3)


def test_transform_brute_force():
    rng = np.random.default_rng(0)
    a = rng.standard_normal((2, 3, 4)).astype(np.float32)
    b = np.zeros_like(a)
    want = np.empty_like(a)
    for idx in np.ndindex(a.shape):
        want[idx] = np.float32(np.float32(1.25) * a[idx]) + np.float32(-0.5)
    oracle.tensor_transform(oracle.TRANSFORM_SCALE_BIAS, [a, b], [1.25, -0.5])
    assert np.array_equal(b, want)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sums_to_statistics_transform_closed_form(dtype):
    """mean = s/n, var = max(q/n - mean^2, 0) * n/(n-1), running = d*old + (1-d)*new
    (batchnorm.cu:297-312) against float64 arithmetic; n == 0 leaves var = 1 (:337-345)."""
    rng = np.random.default_rng(1)
    c, n, decay = 7, 1000, 0.9
    x = rng.standard_normal((n, c))
    s, q = x.sum(0), (x * x).sum(0)
    mean, var = s.astype(dtype).reshape(1, c, 1), q.astype(dtype).reshape(1, c, 1)
    rm, rv = np.full((1, c, 1), 0.5, dtype), np.full((1, c, 1), 2.0, dtype)
    oracle.tensor_transform(oracle.TRANSFORM_SUMS_TO_STATISTICS, [mean, var, rm, rv], [n, decay])
    m64 = s / n
    v64 = np.maximum(q / n - m64 * m64, 0) * n / (n - 1)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.allclose(mean.ravel(), m64, rtol=tol, atol=tol)
    assert np.allclose(var.ravel(), v64, rtol=10 * tol)
    assert np.allclose(var.ravel(), x.var(0, ddof=1), rtol=10 * tol)      # it is the unbiased variance
    assert np.allclose(rm.ravel(), decay * 0.5 + (1 - decay) * m64, rtol=tol, atol=tol)
    assert np.allclose(rv.ravel(), decay * 2.0 + (1 - decay) * v64, rtol=10 * tol)
    mean0, var0 = np.zeros((c,), dtype), np.zeros((c,), dtype)
    rm0, rv0 = np.full(c, 0.5, dtype), np.full(c, 2.0, dtype)
    oracle.tensor_transform(oracle.TRANSFORM_SUMS_TO_STATISTICS, [mean0, var0, rm0, rv0], [0, decay])
    assert (var0 == 1).all() and (mean0 == 0).all() and (rm0 == 0.5).all() and (rv0 == 2.0).all()


@pytest.mark.parametrize("reduce_shape", [(1, 1, 5, 6), (3, 1, 1, 6), (1, 4, 1, 1), (3, 4, 5, 1), (1, 1, 1, 1),
                                          (3, 4, 5, 6)])
def test_reduce_sum_reference_closed_forms(reduce_shape):
    """test_reduce of the reference (:218-300): every reduced cell equals the plain
    sum of its addends; reducing the result again to one cell gives
    (size - 1) * size / 2; the destination is accumulated into, not overwritten."""
    shape = (3, 4, 5, 6)
    src = _offsets(shape)                                   # exact in float64
    dst = np.full(reduce_shape, 10.0)
    oracle.tensor_reduce_sum(src, dst)
    want = np.full(reduce_shape, 10.0)
    for idx in np.ndindex(shape):
        want[tuple(0 if reduce_shape[i] == 1 else idx[i] for i in range(4))] += src[idx]
    assert np.array_equal(dst, want)
    single = np.zeros((1, 1, 1, 1))
    oracle.tensor_reduce_sum(dst - 10.0, single)
    size = src.size
    assert single.item() == (size - 1) * size / 2


def test_reduce_sum_of_squares_and_interior_only():
    rng = np.random.default_rng(3)
    halo = rng.standard_normal((2, 3, 6, 9)).astype(np.float32)
    interior = halo[:, :, 1:5, 2:7]
    dst = np.zeros((1, 3, 1, 1), np.float32)
    oracle.tensor_reduce_sum(interior, dst, square=True)
    want = (interior.astype(np.float64) ** 2).sum(axis=(0, 2, 3))
    assert np.allclose(dst.ravel(), want, rtol=1e-6)
    # the channel sums of batch-norm are this reduction: same numbers as the dedicated oracle function
    x = np.ascontiguousarray(interior)
    s, q = oracle.bn_channel_sums_and_sqsums(x)
    dst2 = np.zeros((1, 3, 1, 1), np.float32)
    oracle.tensor_reduce_sum(interior, dst2)
    assert np.allclose(dst2.ravel(), s, rtol=1e-6) and np.allclose(dst.ravel(), q, rtol=1e-6)

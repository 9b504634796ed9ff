"""Solve / Inverse / Cholesky against the CPU oracle (LAPACK through numpy, as the native backend calls it).

The device kernels use another operation order than LAPACK's blocked routines, so agreement is to rounding: errors are measured
against the conditioning-free residuals (a @ x - b, inv(a) @ a - I, L @ L.T - a) as well as against the oracle's values."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('dt,tol', [('float32', 1e-4), ('float64', 1e-11)])
def test_solve_inverse_cholesky(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(3)
    for n in (1, 2, 5, 33, 130, 300):
        a = (rng.standard_normal((n, n)) + np.sqrt(n) * np.eye(n)).astype(dt)
        a[0], a[n // 2] = a[n // 2].copy(), a[0].copy()  # the largest entries leave the diagonal: pivoting has to act
        for m in (None, 1, 4):
            b = rng.standard_normal((n,) if m is None else (n, m)).astype(dt)
            x = chx.solve(chx.array(a), chx.array(b))
            ref = O.solve(a, b)
            assert x.shape == ref.shape and x.dtype == ref.dtype
            assert_close(x.get(), ref, tol * n, 'solve n=%d m=%r' % (n, m))
            assert np.abs(a.astype(np.float64) @ x.get().astype(np.float64) - b).max() <= tol * n
        inv = chx.inv(chx.array(a))
        assert_close(inv.get(), O.inv(a), tol * n, 'inv n=%d' % n)
        assert np.abs(inv.get().astype(np.float64) @ a - np.eye(n)).max() <= tol * n
        spd = (a.astype(np.float64) @ a.T.astype(np.float64)).astype(dt)
        low = chx.cholesky(chx.array(spd)).get()
        assert_close(low, O.cholesky(spd), tol * n, 'cholesky n=%d' % n)
        assert np.array_equal(low, np.tril(low)), 'strict upper triangle must be zero'
        spoiled = np.tril(spd) + np.triu(rng.standard_normal((n, n)).astype(dt), 1)
        assert np.array_equal(chx.cholesky(chx.array(spoiled)).get(), low), 'only the lower triangle is read'
    # views and mixed dtypes: a transposed view, an integer matrix (computes in float32), float32 with float64 (float64)
    a = (rng.standard_normal((6, 6)) + 3 * np.eye(6)).astype(dt)
    b = rng.standard_normal((6, 2)).astype(dt)
    assert_close(chx.solve(chx.array(a).T, chx.array(b)).get(), O.solve(a.T, b), tol * 10, 'transposed view')
    ai = np.array([[2, 1], [1, 3]], np.int32)
    assert_close(chx.inv(chx.array(ai)).get(), O.inv(ai), 1e-5, 'integer input')
    x = chx.solve(chx.array(a.astype('float32')), chx.array(b.astype('float64')))
    assert x.dtype == np.float64


def test_linalg_errors_and_empty():
    import chainer_amd as chx
    singular = np.array([[1., 2., 3.], [2., 4., 6.], [1., 0., 1.]], 'float32')
    with pytest.raises(chx.ChainerxError):
        chx.solve(chx.array(singular), chx.array(np.ones(3, 'float32')))
    with pytest.raises(chx.ChainerxError):
        chx.inv(chx.array(np.zeros((4, 4), 'float64')))
    with pytest.raises(chx.ChainerxError):
        chx.cholesky(chx.array(np.array([[1., 2.], [2., 1.]], 'float32')))  # indefinite
    with pytest.raises(chx.DimensionError):
        chx.inv(chx.zeros((2, 3), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.cholesky(chx.zeros((2, 2, 2), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.solve(chx.zeros((3, 3), 'float32'), chx.zeros((2,), 'float32'))
    for fn in (chx.inv, chx.cholesky):
        with pytest.raises(chx.DtypeError):
            fn(chx.zeros((2, 2), 'float16'))
    with pytest.raises(chx.DtypeError):
        chx.solve(chx.zeros((2, 2), 'float16'), chx.zeros((2,), 'float16'))
    assert chx.inv(chx.zeros((0, 0), 'float32')).shape == (0, 0)
    assert chx.solve(chx.zeros((0, 0), 'float32'), chx.zeros((0, 2), 'float32')).shape == (0, 2)

"""FixedBatchNorm, MaxPool, AveragePool, Take and the LSTM cell against the CPU oracle."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, channels_last
from test_oracle_pins import BN_GRID, POOL_GRID

pytestmark = pytest.mark.gpu

DT = [('float32', 1e-5), ('float16', 2e-2), ('float64', 1e-12)]


@pytest.mark.parametrize('dt,tol', DT)
def test_fixed_batch_norm(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(0)
    for shape in [(2, 16, 5, 7), (3, 64, 8, 8), (2, 5, 3, 3), (1, 8, 1, 1), (4, 32, 14, 14), (8, 64, 7, 7), (3, 2000, 2, 2), (2, 700, 1, 3), (2, 3, 70, 70)]:
        C = shape[1]
        x = rng.standard_normal(shape).astype(dt)
        g = rng.uniform(0.5, 1.5, C).astype(dt)
        b, m = rng.standard_normal(C).astype(dt), rng.standard_normal(C).astype(dt)
        v = rng.uniform(0.5, 1.5, C).astype(dt)
        P = [chx.array(a) for a in (g, b, m, v)]
        x2 = np.concatenate([x, x], 3)
        for lay, X, xr in (('nchw', chx.array(x), x), ('nhwc', channels_last(chx, x), x), ('strided', chx.array(x2)[:, :, :, ::2], x2[:, :, :, ::2])):
            ref = O.fixed_batch_norm(xr, g, b, m, v, 2e-5, (0, 2, 3))
            y = chx.fixed_batch_norm(X, *P, 2e-5, (0, 2, 3))
            assert_close(y.get(), ref, tol, 'bn %s %s %s' % (dt, lay, shape))


@pytest.mark.parametrize('xs,rs,axis', BN_GRID)
def test_fixed_batch_norm_reference_grid(xs, rs, axis):
    """tests/chainerx_tests/unit_tests/routines_tests/test_normalization.py:50-58: every axis convention."""
    import chainer_amd as chx
    rng = np.random.default_rng(1)
    for dt, tol in DT:
        x = rng.standard_normal(xs).astype(dt)
        g, b, m = [rng.standard_normal(rs).astype(dt) for _ in range(3)]
        v = rng.uniform(0.5, 1.5, rs).astype(dt)
        y = chx.fixed_batch_norm(chx.array(x), *[chx.array(a) for a in (g, b, m, v)], 1e-3, axis)
        assert_close(y.get(), O.fixed_batch_norm(x, g, b, m, v, 1e-3, axis), tol)
    with pytest.raises(chx.DimensionError):
        chx.fixed_batch_norm(chx.array(x), *[chx.zeros((3,), dt) for _ in range(4)], 1e-3, axis)
    with pytest.raises(chx.DtypeError):
        chx.fixed_batch_norm(chx.zeros((2, 3), 'int32'), *[chx.zeros((3,), 'float32') for _ in range(4)])


@pytest.mark.parametrize('dt,tol', DT)
def test_pooling(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(2)
    cases = [((2, 16, 9, 8), 3, 2, 1, False), ((2, 16, 9, 8), 3, 2, 1, True), ((2, 3, 7, 7), 2, 2, 0, False), ((1, 8, 7, 7), 7, 1, 0, False),
             ((2, 64, 12, 12), (3, 2), (2, 1), (1, 0), True), ((2, 8, 112, 112), 3, 2, 1, False), ((2, 8, 32, 32), 2, 2, 0, False),
             ((1, 4, 16, 24), 3, 2, 1, True), ((1, 4, 16, 16), (2, 3), 2, (0, 1), False)]
    # whole-plane windows (global pooling) over more planes than one workgroup takes, odd and even plane sizes
    cases += [((3, 200, 7, 7), 7, 1, 0, False), ((2, 301, 5, 5), 5, 1, 0, False), ((2, 130, 6, 6), 6, 1, 0, False), ((1, 257, 3, 5), (3, 5), 1, 0, False),
              ((2, 150, 8, 8), 8, 1, 0, False), ((1, 512, 2, 2), 2, 1, 0, False)]  # full workgroups of even planes
    cases += [(xs, k, s, p, cv) for (xs, k, s, p) in POOL_GRID for cv in (False, True)]
    for shape, k, s, p, cv in cases:
        x = rng.standard_normal(shape).astype(dt)
        for lay, X in (('nchw', chx.array(x)), ('nhwc', channels_last(chx, x))):
            what = '%s %s %s' % (dt, lay, (shape, k, s, p, cv))
            assert_exact(chx.max_pool(X, k, s, p, cv).get(), O.max_pool(x, k, s, p, cv), 'max_pool ' + what)
            if not cv:
                for mode in ('zero', 'ignore'):
                    got, ref = chx.average_pool(X, k, s, p, mode).get(), O.average_pool(x, k, s, p, mode)
                    fin = np.isfinite(ref)  # 'ignore' windows that lie entirely in the padding are 0/0
                    assert np.array_equal(np.isnan(got), np.isnan(ref))
                    assert_close(np.where(fin, got, 0), np.where(fin, ref, 0), tol * 2, 'average_pool %s %s' % (mode, what))


def test_pooling_special_values_and_dtypes():
    import chainer_amd as chx
    rng = np.random.default_rng(3)
    xi = rng.integers(-50, 50, (2, 4, 6, 6)).astype('int32')
    assert_exact(chx.max_pool(chx.array(xi), 3, 2, 1).get(), O.max_pool(xi, 3, 2, 1), 'int32 max_pool')
    xn = rng.standard_normal((1, 8, 6, 6)).astype('float32')
    xn[0, 3, 2, 2] = np.nan
    assert_exact(chx.max_pool(channels_last(chx, xn), 3, 1, 1).get(), O.max_pool(xn, 3, 1, 1), 'NaN propagates like AMax')
    with pytest.raises(chx.DtypeError):
        chx.average_pool(chx.array(xi), 2)


@pytest.mark.parametrize('dt', ['float32', 'float16', 'int8', 'int64', 'bool', 'float64'])
def test_take(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(4)
    a = (rng.standard_normal((50, 24)) * 10).astype(dt)
    A = chx.array(a)
    for idt in ('int32', 'int64', 'uint8', 'int8'):
        idx = rng.integers(0, 50, (7, 3)).astype(idt)
        assert_exact(chx.take(A, chx.array(idx), 0).get(), O.take(a, idx, 0), 'axis 0 %s' % idt)
        idx1 = rng.integers(0, 24, (5,)).astype(idt)
        assert_exact(chx.take(A, chx.array(idx1), 1).get(), O.take(a, idx1, 1), 'axis 1 %s' % idt)
    neg = np.array([0, -1, -50, 49, 3], 'int64')
    assert_exact(chx.take(A, chx.array(neg), 0).get(), O.take(a, neg, 0), 'negative indices')
    wr = np.array([0, 14, 3, 1, -10, 1, 1000, -1000], 'int64')
    assert_exact(chx.take(A, chx.array(wr), 1, 'wrap').get(), O.take(a, wr, 1, 'wrap'), 'wrap')
    assert_exact(chx.take(A, chx.array(wr), 1, 'clip').get(), O.take(a, wr, 1, 'clip'), 'clip')
    assert_exact(chx.take(A.T, chx.array(neg[:3] % 24), 0).get(), O.take(a.T, neg[:3] % 24, 0), 'transposed source')
    empty = chx.take(A, chx.array(np.zeros((0,), 'int64')), 0)
    assert empty.shape == (0, 24)


def test_take_bounds_and_embedding_shape():
    import chainer_amd as chx
    rng = np.random.default_rng(5)
    # native raises in the default mode (CX/native/native_device/indexing.cc:68-74); here the call itself returns (no wait for the
    # device) and the error surfaces at the first point where the result could be read
    bad = chx.take(chx.zeros((4, 3), 'float32'), chx.array(np.array([5], 'int64')), 0)
    with pytest.raises(IndexError, match='Index 5 is out of bounds for axis 0 with size 4'):
        bad.get()
    assert bad.get().shape == (1, 3)  # reported once: the record is cleared
    bad = chx.take(chx.zeros((4, 3), 'float32'), chx.array(np.array([[0, -5]], 'int32')), 0)
    good = chx.take(chx.ones((4, 3), 'float32'), chx.array(np.array([1], 'int64')), 0)  # later, valid work does not clear it
    with pytest.raises(IndexError):
        chx.synchronize()
    chx.synchronize()
    assert_exact(good.get(), np.ones((1, 3), 'float32'), 'a valid take after a bad one')
    with pytest.raises(IndexError):  # 'raise' checks inside the call
        chx.take(chx.zeros((4, 3), 'float32'), chx.array(np.array([-5], 'int64')), 0, 'raise')
    chx.synchronize()  # ... and leaves nothing behind
    with pytest.raises(chx.DtypeError):
        chx.take(chx.zeros((4, 3), 'float32'), chx.zeros((2,), 'float32'), 0)
    ids = rng.integers(0, 10000, (128, 35)).astype('int32')
    W = rng.standard_normal((10000, 650)).astype('float32')
    Wd, Id = chx.array(W), chx.array(ids)
    assert_exact(chx.take(Wd, Id[:, 3], 0).get(), W[ids[:, 3]], 'embedding rows, strided ids')
    assert_exact(chx.take(Wd, Id, 0).get(), W[ids], 'embedding rows, the whole [128,35] batch')
    with pytest.raises(IndexError):
        chx.take(Wd, chx.array(np.array([3, 10000], 'int64')), 0).get()
    # long rows in 4-byte pieces (68 bytes) and in 16-byte pieces (2048 bytes), negative and wrapped indices
    for shape, dt in (((300, 17), 'float32'), ((90, 1024), 'float16'), ((40, 33), 'int32')):
        a = (rng.standard_normal(shape) * 100).astype(dt)
        idx = rng.integers(-shape[0], shape[0], (9, 11)).astype('int64')
        assert_exact(chx.take(chx.array(a), chx.array(idx), 0).get(), O.take(a, idx, 0), 'rows %r' % (shape,))
        far = rng.integers(-5 * shape[0], 5 * shape[0], (70,)).astype('int64')
        assert_exact(chx.take(chx.array(a), chx.array(far), 0, 'wrap').get(), O.take(a, far, 0, 'wrap'), 'wrapped rows %r' % (shape,))


@pytest.mark.parametrize('dt,tol', [('float32', 1e-5), ('float64', 1e-12), ('float16', 2e-2)])
def test_lstm_cell(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(6)
    c = rng.standard_normal((16, 24)).astype(dt)
    g = rng.standard_normal((16, 96)).astype(dt)
    h1, c1 = chx.lstm(chx.array(c), chx.array(g))
    h2, c2 = O.lstm(c, g)
    assert_close(h1.get(), h2, tol, 'h')
    assert_close(c1.get(), c2, tol, 'c')
    with pytest.raises(chx.DimensionError):
        chx.lstm(chx.array(c), chx.array(g[:, :95]))

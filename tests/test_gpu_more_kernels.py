"""The further elementwise kernels (unary math, Square / Abs / Sign, predicates, logical ops, Power, Fmod, Arctan2, Where) and
the AMin / ArgMin / All / Any reductions against the CPU oracle.

Bar: bit-exact wherever the result is a selection, a comparison, an integer operation or one IEEE operation; the libm-class
functions are held to the float tolerance of the contract (1e-5 float32, 2e-2 float16; 1e-12 float64)."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, padded, upload_view

pytestmark = pytest.mark.gpu

ALL = ['bool', 'int8', 'int16', 'int32', 'int64', 'uint8', 'float16', 'float32', 'float64']
NUMERIC = ALL[1:]
FLOATS = ['float16', 'float32', 'float64']

# name -> sampler of valid arguments
UNARY_DOMAINS = {
    'erf': lambda r, s: r.standard_normal(s) * 2, 'expm1': lambda r, s: r.standard_normal(s) * 3, 'exp2': lambda r, s: r.standard_normal(s) * 5,
    'log10': lambda r, s: r.random(s) * 100 + 1e-3, 'log2': lambda r, s: r.random(s) * 100 + 1e-3, 'log1p': lambda r, s: r.random(s) * 10 - 0.9,
    'sinh': lambda r, s: r.standard_normal(s) * 3, 'cosh': lambda r, s: r.standard_normal(s) * 3, 'arcsinh': lambda r, s: r.standard_normal(s) * 50,
    'arccosh': lambda r, s: r.random(s) * 50 + 1, 'sin': lambda r, s: r.standard_normal(s) * 3, 'cos': lambda r, s: r.standard_normal(s) * 3,
    'tan': lambda r, s: r.random(s) * 2.6 - 1.3, 'arcsin': lambda r, s: r.random(s) * 1.98 - 0.99, 'arccos': lambda r, s: r.random(s) * 1.98 - 0.99,
    'arctan': lambda r, s: r.standard_normal(s) * 10,
}


def rand(rng, shape, dt):
    if dt == 'bool':
        return rng.random(shape) > 0.5
    if np.dtype(dt).kind == 'f':
        return (rng.standard_normal(shape) * 10).astype(dt)
    return rng.integers(0 if dt == 'uint8' else -100, 100, shape).astype(dt)


@pytest.mark.parametrize('dt', FLOATS)
def test_unary_math(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(21)
    tol = {'float16': 2e-3, 'float32': 2e-6, 'float64': 1e-13}[dt]
    for name, sample in UNARY_DOMAINS.items():
        x = sample(rng, (33, 257)).astype(dt)
        assert_close(getattr(chx, name)(chx.array(x)).get(), getattr(O, name)(x), tol, '%s %s' % (name, dt))
    x = (rng.standard_normal((33, 257)) * 5).astype(dt)
    x[0, :8] = [0.5, -0.5, 1.5, -1.5, 2.0, -0.0, np.inf, np.nan]
    for name in ('ceil', 'floor'):  # exact
        assert_exact(getattr(chx, name)(chx.array(x)).get(), getattr(O, name)(x), name)
        assert_exact(getattr(chx, name)(chx.array(x)[:, 1::3]).get(), getattr(O, name)(x[:, 1::3]), name + ' strided')
    # integer inputs are computed in float32 (GetMathResultDtype)
    xi = rng.integers(0, 5, (4, 9)).astype('int32')
    got = chx.sin(chx.array(xi)).get()
    assert got.dtype == np.float32
    assert_close(got, O.sin(xi.astype('float32')), 2e-6, 'sin of int32')


def test_unary_special_values():
    import chainer_amd as chx
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5, 1e-30, 80.0], np.float32)
    with np.errstate(all='ignore'):
        for name in list(UNARY_DOMAINS) + ['ceil', 'floor']:
            got, ref = getattr(chx, name)(chx.array(x)).get(), getattr(O, name)(x)
            assert np.array_equal(np.isnan(got), np.isnan(ref)), name
            assert np.array_equal(np.isinf(got), np.isinf(ref)) and np.array_equal(got[np.isinf(ref)], ref[np.isinf(ref)]), name
            fin = np.isfinite(ref)
            assert np.allclose(got[fin], ref[fin], rtol=1e-5, atol=1e-37), name


@pytest.mark.parametrize('dt', NUMERIC)
def test_square_abs_sign(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(22)
    x = rand(rng, (19, 131), dt)
    if np.dtype(dt).kind == 'f':
        x[0, :5] = [np.nan, -0.0, 0.0, np.inf, -np.inf]
    else:
        info = np.iinfo(dt)
        x[0, :3] = [info.min, info.max, 0]  # wrap-around cases of the integer forms
    X = chx.array(x)
    with np.errstate(all='ignore'):
        assert_exact(chx.square(X).get(), O.square(x), 'square')
        assert_exact(chx.absolute(X).get(), O.absolute(x), 'absolute')
        assert_exact(chx.sign(X).get(), O.sign(x), 'sign')
        assert_exact(chx.sign(X.T[::2]).get(), O.sign(x.T[::2]), 'sign of a view')
    for f in (chx.square, chx.absolute, chx.sign):
        with pytest.raises(chx.DtypeError):
            f(chx.array(np.zeros(3, bool)))


@pytest.mark.parametrize('dt', ALL)
def test_predicates_and_logical(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(23)
    x, y = rand(rng, (23, 67), dt), rand(rng, (23, 67), dt)
    x[x == 7] = 0
    if np.dtype(dt).kind == 'f':
        x[1, :4] = [np.nan, np.inf, -np.inf, -0.0]
    X, Y = chx.array(x), chx.array(y)
    for name in ('logical_not', 'isnan', 'isinf', 'isfinite'):
        got = getattr(chx, name)(X).get()
        assert got.dtype == np.bool_
        assert_exact(got, getattr(O, name)(x), name)
    for name in ('logical_and', 'logical_or', 'logical_xor'):
        assert_exact(getattr(chx, name)(X, Y).get(), getattr(O, name)(x, y), name)
        assert_exact(getattr(chx, name)(X[::2, 1::3], Y[::2, 1::3]).get(), getattr(O, name)(x[::2, 1::3], y[::2, 1::3]), name + ' views')
    assert_exact(chx.less(X, Y).get(), x < y, 'less')
    assert_exact(chx.less_equal(X, Y).get(), x <= y, 'less_equal')
    other = chx.array(np.ones((23, 67), 'int32' if dt == 'bool' else 'bool'))
    with pytest.raises(chx.DtypeError):
        chx.logical_and(X, other)


@pytest.mark.parametrize('dt', NUMERIC)
def test_power(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(24)
    if np.dtype(dt).kind == 'f':
        x = (rng.random((17, 41)) * 4 + 0.1).astype(dt)
        e = (rng.standard_normal((17, 41)) * 2).astype(dt)
        tol = {'float16': 2e-3, 'float32': 2e-6, 'float64': 1e-13}[dt]
        assert_close(chx.power(chx.array(x), chx.array(e)).get(), O.power(x, e), tol, 'power')
        assert_close(chx.power(chx.array(x), 2.5).get(), O.power(x, np.asarray(2.5, dt)), tol, 'power AS')
        assert_close(chx.power(2.0, chx.array(e)).get(), O.power(np.asarray(2.0, dt), e), tol, 'power SA')
    else:
        lo = 0 if dt == 'uint8' else -6
        x = rng.integers(lo, 7, (17, 41)).astype(dt)
        e = rng.integers(lo, 9, (17, 41)).astype(dt)  # negative exponents and results that wrap
        assert_exact(chx.power(chx.array(x), chx.array(e)).get(), O.power(x, e), 'power')
        assert_exact(chx.power(chx.array(x), 3).get(), O.power(x, np.asarray(3, dt)), 'power AS')
        assert_exact(chx.power(3, chx.array(e)).get(), O.power(np.asarray(3, dt), e), 'power SA')
        assert_exact(chx.power(chx.array(x).T, chx.array(e).T).get(), O.power(x.T, e.T), 'power of views')
    with pytest.raises(chx.DtypeError):
        chx.power(chx.array(np.ones(3, bool)), chx.array(np.ones(3, bool)))


@pytest.mark.parametrize('dt', FLOATS)
def test_fmod_arctan2(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(25)
    x = (rng.standard_normal((29, 53)) * 10).astype(dt)
    y = (rng.standard_normal((29, 53)) * 3).astype(dt)
    y[np.abs(y) < 0.05] = 1
    tol = {'float16': 2e-3, 'float32': 2e-6, 'float64': 1e-13}[dt]
    assert_exact(chx.fmod(chx.array(x), chx.array(y)).get(), O.fmod(x, y), 'fmod')  # fmod is exact
    assert_close(chx.arctan2(chx.array(x), chx.array(y)).get(), O.arctan2(x, y), tol, 'arctan2')
    b = y[0]
    assert_close(chx.arctan2(chx.array(x), chx.array(b)).get(), O.arctan2(x, np.broadcast_to(b, x.shape)), tol, 'arctan2 broadcast')
    with pytest.raises(chx.DtypeError):
        chx.fmod(chx.array(np.ones(3, 'int32')), chx.array(np.ones(3, 'int32')))


@pytest.mark.parametrize('dt', ALL)
def test_where(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(26)
    c = rng.random((31, 45)) > 0.4
    x, y = rand(rng, (31, 45), dt), rand(rng, (31, 45), dt)
    C, X, Y = chx.array(c), chx.array(x), chx.array(y)
    assert_exact(chx.where(C, X, Y).get(), O.where(c, x, y, dt), 'where AAA')
    assert_exact(chx.where(C.T, X.T, Y.T).get(), O.where(c.T, x.T, y.T, dt), 'where of transposed views')
    assert_exact(chx.where(C[::2, 3:40:2], X[::2, 3:40:2], Y[::2, 3:40:2]).get(), O.where(c[::2, 3:40:2], x[::2, 3:40:2], y[::2, 3:40:2], dt), 'sliced')
    # broadcasting of the condition (a column) and of y (a row)
    assert_exact(chx.where(C[:, :1], X, Y[:1]).get(), O.where(np.broadcast_to(c[:, :1], x.shape), x, np.broadcast_to(y[:1], x.shape), dt), 'broadcast')
    if dt != 'bool':
        s = 3 if np.dtype(dt).kind != 'f' else 1.5
        assert_exact(chx.where(C, X, s).get(), O.where(c, x, s, dt), 'where AAS')
        assert_exact(chx.where(C, s, Y).get(), O.where(c, s, y, dt), 'where ASA')
        sd = np.dtype('float32') if isinstance(s, float) else np.dtype('int32')
        got = chx.where(C, s, 2 * s)
        assert got.dtype == sd
        assert_exact(got.get(), O.where(c, s, 2 * s, sd), 'where ASS')
    # a non-bool condition is cast to bool first
    ci = rng.integers(-1, 2, (31, 45)).astype('int32')
    assert_exact(chx.where(chx.array(ci), X, Y).get(), O.where(ci, x, y, dt), 'int condition')
    # mixed dtypes promote by the ChainerX rule: a float operand decides, the wider float wins (CX/dtype.h PromoteTypes)
    z = rand(rng, (31, 45), 'float32')
    rdt = np.dtype('float64' if dt == 'float64' else 'float32')
    got = chx.where(C, X, chx.array(z))
    assert got.dtype == rdt
    assert_exact(got.get(), O.where(c, x, z, rdt), 'promotion')


@pytest.mark.parametrize('dt', ALL)
def test_amin_argmin_all_any(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(27)
    for shape, axis in [((7, 300), 1), ((7, 300), 0), ((5, 6, 70), (0, 2)), ((4, 5000), 1), ((3, 4, 5), None), ((2, 70000), 1)]:
        x = rand(rng, shape, dt)
        X = chx.array(x)
        assert_exact(chx.amin(X, axis).get(), O.amin(x, axis), 'amin %r %r' % (shape, axis))
        assert_exact(chx.amin(X, axis, True).get(), O.amin(x, axis, True), 'amin keepdims')
        if axis is None or isinstance(axis, int):
            assert_exact(chx.argmin(X, axis).get(), O.argmin(x, axis), 'argmin %r %r (ties follow the native tree)' % (shape, axis))
        assert_exact(chx.all(X, axis).get(), O.all(x, axis), 'all')
        assert_exact(chx.any(X, axis).get(), O.any(x, axis), 'any')
        assert_exact(chx.all(X, axis, True).get(), O.all(x, axis, True), 'all keepdims')
    # all-true / all-false rows
    z = np.zeros((3, 1000), dt)
    z[1] = 1
    z[2, 777] = 1
    assert_exact(chx.all(chx.array(z), 1).get(), np.array([False, True, False]), 'all rows')
    assert_exact(chx.any(chx.array(z), 1).get(), np.array([False, True, True]), 'any rows')
    # padded parent (non-contiguous)
    xp = padded((4, 3, 5), rand(rng, (4, 3, 5), dt), 1, dt)
    assert_exact(chx.amin(upload_view(chx, xp), (0, 2)).get(), O.amin(xp, (0, 2)), 'amin padded')
    with pytest.raises(chx.DimensionError):
        chx.amin(chx.array(np.zeros((3, 0), dt)), 1)
    with pytest.raises(chx.DimensionError):
        chx.argmin(chx.array(np.zeros((3, 0), dt)), 1)


def test_amin_argmin_nan_rule():
    """NaN propagates through AMin; ArgMin never lets a NaN replace the accumulator and never replaces a leading NaN."""
    import chainer_amd as chx
    rng = np.random.default_rng(28)
    x = rng.standard_normal((6, 500)).astype('float32')
    x[1, 123] = np.nan
    x[2, 0] = np.nan
    x[3, 40:45] = x[3].min() - 1  # a five-way tie inside one block of the tree
    x[4, [10, 300]] = x[4].min() - 1  # a tie across blocks
    X = chx.array(x)
    assert_exact(chx.amin(X, 1).get(), O.amin(x, 1), 'amin with NaN')
    assert_exact(chx.argmin(X, 1).get(), O.argmin(x, 1), 'argmin with NaN and ties')
    assert np.isnan(chx.amin(X, 1).get()[1])


@pytest.mark.parametrize('dt', NUMERIC)
def test_floor_divide_mod(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(29)
    x, y = rand(rng, (23, 77), dt), rand(rng, (23, 77), dt)
    y[0, :5] = 0  # zero divisors
    x[1, :5] = 0
    X, Y = chx.array(x), chx.array(y)
    s = 3 if np.dtype(dt).kind != 'f' else 2.5
    sv = np.asarray(s, dt)
    with np.errstate(all='ignore'):
        for name in ('floor_divide', 'mod'):
            f, g = getattr(chx, name), getattr(O, name)
            assert_exact(f(X, Y).get(), g(x, y), name)
            assert_exact(f(X, s).get(), g(x, sv), name + ' AS')
            assert_exact(f(s, Y).get(), g(sv, y), name + ' SA')
            assert_exact(f(X.T[::2], Y.T[::2]).get(), g(x.T[::2], y.T[::2]), name + ' views')
            assert_exact(f(X, Y[:1]).get(), g(x, np.broadcast_to(y[:1], x.shape)), name + ' broadcast')
    with pytest.raises(chx.DtypeError):
        chx.floor_divide(chx.array(np.ones(3, bool)), chx.array(np.ones(3, bool)))


@pytest.mark.parametrize('dt', ['bool', 'int8', 'int16', 'int32', 'int64', 'uint8'])
def test_bitwise_and_shifts(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(30)
    x, y = rand(rng, (19, 65), dt), rand(rng, (19, 65), dt)
    X, Y = chx.array(x), chx.array(y)
    for name in ('bitwise_and', 'bitwise_or', 'bitwise_xor'):
        f, g = getattr(chx, name), getattr(O, name)
        assert_exact(f(X, Y).get(), g(x, y), name)
        assert_exact(f(X[::2, 1::3], Y[::2, 1::3]).get(), g(x[::2, 1::3], y[::2, 1::3]), name + ' views')
        sc = True if dt == 'bool' else 5
        assert_exact(f(X, sc).get(), g(x, np.asarray(sc, dt)), name + ' AS')
        assert_exact(f(sc, X).get(), g(x, np.asarray(sc, dt)), name + ' SA swaps')
    with pytest.raises(chx.DtypeError):
        chx.bitwise_and(chx.array(np.ones(3, 'float32')), chx.array(np.ones(3, 'float32')))
    if dt == 'bool':
        with pytest.raises(chx.DtypeError):
            chx.left_shift(X, Y)
        return
    bits = np.dtype(dt).itemsize * 8
    cnt = rng.integers(0, bits, (19, 65)).astype(dt)
    Cn = chx.array(cnt)
    assert_exact(chx.left_shift(X, Cn).get(), O.left_shift(x, cnt), 'left_shift')
    assert_exact(chx.right_shift(X, Cn).get(), O.right_shift(x, cnt), 'right_shift')
    assert_exact(chx.left_shift(X, 3).get(), O.left_shift(x, np.asarray(3, dt)), 'left_shift AS')
    assert_exact(chx.right_shift(X, 2).get(), O.right_shift(x, np.asarray(2, dt)), 'right_shift AS')
    got = chx.left_shift(3, Cn)  # Scalar << Array is int64
    assert got.dtype == np.int64
    assert_exact(got.get(), O.left_shift(np.full(cnt.shape, 3, np.int64), cnt.astype(np.int64)), 'left_shift SA')
    assert_exact(chx.right_shift(-1000, Cn).get(), O.right_shift(np.full(cnt.shape, -1000, np.int64), cnt.astype(np.int64)), 'right_shift SA')


@pytest.mark.parametrize('dt', ALL)
def test_creation_patterns(dt):
    import chainer_amd as chx
    for n in (0, 1, 5, 33):
        assert_exact(chx.identity(n, dt).get(), O.identity(n, dt), 'identity %d' % n)
    for (n, m, k) in [(4, 4, 0), (5, 7, 2), (7, 5, -3), (6, 6, 9), (6, 6, -9), (1, 9, 3), (40, 37, 1)]:
        assert_exact(chx.eye(n, m, k, dt).get(), O.eye(n, m, k, dt), 'eye %r' % ((n, m, k),))
        assert_exact(chx.tri(n, m, k, dt).get(), O.tri(n, m, k, dt), 'tri %r' % ((n, m, k),))
    rng = np.random.default_rng(31)
    v = rand(rng, (6,), dt)
    for k in (0, 2, -3):
        assert_exact(chx.diagflat(chx.array(v), k).get(), O.diagflat(v, k), 'diagflat k=%d' % k)
    v2 = rand(rng, (2, 3), dt)
    assert_exact(chx.diagflat(chx.array(v2)[:, ::-1], 1).get(), O.diagflat(v2[:, ::-1], 1), 'diagflat of a view')
    m2 = rand(rng, (5, 7), dt)
    for k in (0, 2, -1, 6, -5):
        assert_exact(chx.diag(chx.array(m2), k).get(), np.diag(m2, k), 'diag view k=%d' % k)
    if dt != 'bool':
        for (a, b, num, ep) in [(0, 10, 11, True), (-3, 7.5, 50, True), (2, -2, 9, False), (5, 5, 1, True), (0, 1, 4097, True)]:
            assert_exact(chx.linspace(a, b, num, ep, dt).get(), O.linspace(a, b, num, ep, dt), 'linspace %r' % ((a, b, num, ep),))
    assert chx.linspace(0, 1, 0).shape == (0,)
    with pytest.raises(chx.DimensionError):
        chx.eye(-1)


@pytest.mark.parametrize('dt', ALL)
def test_cumsum_nansum(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(32)
    for shape, axis in [((7, 130), 1), ((7, 130), 0), ((4, 5, 6), 1), ((3, 4, 5), None), ((2000,), 0), ((5, 9), -1)]:
        x = rand(rng, shape, dt)
        got = chx.cumsum(chx.array(x), axis).get()
        assert_exact(got, O.cumsum(x, axis), 'cumsum %r axis %r (serial order: bit-exact)' % (shape, axis))
    xv = rand(rng, (9, 40), dt)
    assert_exact(chx.cumsum(chx.array(xv).T[::2], 1).get(), O.cumsum(xv.T[::2], 1), 'cumsum of a view')
    if np.dtype(dt).kind == 'f':
        x = rand(rng, (6, 300), dt)
        x[x > 15] = np.nan
        assert np.isnan(x).any()
        assert_close(chx.nansum(chx.array(x), 1).get(), O.nansum(x, 1), None, 'nansum')
        assert_close(chx.nansum(chx.array(x)).get(), O.nansum(x), None, 'nansum all axes')


@pytest.mark.parametrize('dt', ALL)
def test_add_at(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(33)
    a = rand(rng, (5, 6, 7), dt)
    for axis, ishape in [(0, (4,)), (1, (3, 2)), (2, (9,)), (1, (1,))]:
        dim = a.shape[axis]
        idx = rng.integers(-dim, dim, ishape)  # repeated and negative indices
        b = rand(rng, a.shape[:axis] + ishape + a.shape[axis + 1:], dt)
        got = chx.add_at(chx.array(a), chx.array(idx), axis, chx.array(b)).get()
        assert_exact(got, O.add_at(a, idx, axis, b), 'add_at axis %d %r' % (axis, ishape))
        big = idx * 5
        for mode in ('wrap', 'clip'):
            assert_exact(chx.add_at(chx.array(a), chx.array(big.astype('int32')), axis, chx.array(b), mode).get(),
                         O.add_at(a, big, axis, b, mode), 'add_at %s' % mode)
    # views on both sides
    idx = np.array([1, 1, 0, 3])
    b = rand(rng, (5, 4, 7), dt)
    got = chx.add_at(chx.array(a)[:, ::-1], chx.array(idx), 1, chx.array(b)[::-1]).get()
    assert_exact(got, O.add_at(a[:, ::-1], idx, 1, b[::-1]), 'add_at views')
    with pytest.raises(chx.ChainerxIndexError):  # default mode: raised where the result would be read
        chx.add_at(chx.array(a), chx.array(np.array([6])), 1, chx.array(rand(rng, (5, 1, 7), dt))).get()
    with pytest.raises(chx.ChainerxIndexError):
        chx.add_at(chx.array(a), chx.array(np.array([6])), 1, chx.array(rand(rng, (5, 1, 7), dt)), 'raise')
    # the embedding gradient: many rows scattered into a table
    if dt == 'float32':
        table = np.zeros((50, 16), dt)
        ids = rng.integers(0, 50, (300,))
        g = rng.standard_normal((300, 16)).astype(dt)
        assert_exact(chx.add_at(chx.array(table), chx.array(ids), 0, chx.array(g)).get(), O.add_at(table, ids, 0, g), 'embedding gradient')

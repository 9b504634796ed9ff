"""Sum / AMax / ArgMax / log_softmax against the CPU oracle.

Bar: ArgMax and AMax bit-exact (including the native backend's tie and NaN rules); Sum bit-exact as well, because the
kernels reproduce the native pairwise tree (integers are exact in any order); log_softmax within the float tolerance."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, padded, upload_view

pytestmark = pytest.mark.gpu

SHAPES_AXES = [((5, 70), 1), ((5, 70), 0), ((5, 70), None), ((3, 4, 5), (0, 2)), ((3, 4, 5), 1), ((7, 300), 1), ((4, 1024), 1),
               ((3, 4100), 1), ((2, 70000), 1), ((6,), 0), ((2, 3, 1500), (1, 2)), ((1, 65536 * 3 + 5), 1), ((300, 9), 0),
               ((2, 2, 2, 2), (1, 3)), ((3, 33), 1), ((3, 35), 1), ((3, 3), 1)]
DTYPES = ['float32', 'float64', 'float16', 'int32', 'int64', 'int8', 'uint8', 'bool', 'int16']


def rand(rng, shape, dt):
    if dt == 'bool':
        return rng.random(shape) > 0.7
    if dt.startswith('float'):
        return rng.standard_normal(shape).astype(dt)
    return rng.integers(0 if dt == 'uint8' else -100, 100, shape).astype(dt)


@pytest.mark.parametrize('dt', DTYPES)
def test_reductions_match_oracle(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(0)
    for shape, axis in SHAPES_AXES:
        x = rand(rng, shape, dt)
        X = chx.array(x)
        what = '%s %s axis=%s' % (dt, shape, axis)
        for keep in (False, True):
            assert_exact(chx.sum(X, axis, keep).get(), O.sum(x, axis, keep), 'sum ' + what)
            assert_exact(chx.amax(X, axis, keep).get(), O.amax(x, axis, keep), 'amax ' + what)
        assert_exact(chx.argmax(X, axis).get(), O.argmax(x, axis), 'argmax ' + what)
    if dt != 'bool':  # strided views
        x = (rng.standard_normal((6, 2100)) * 10).astype(dt)
        X = chx.array(x)
        assert_exact(chx.sum(X.T, 0).get(), O.sum(x.T, 0), 'sum of a transposed view')
        assert_exact(chx.argmax(X[:, 3:2051], 1).get(), O.argmax(x[:, 3:2051], 1), 'argmax of a slice')
        assert_exact(chx.argmax(X[:, ::2], 1).get(), O.argmax(x[:, ::2], 1), 'argmax with a step')
        xp = padded((3, 4, 5), rand(rng, (3, 4, 5), dt), 1, dt)
        assert_exact(chx.amax(upload_view(chx, xp), (0, 2)).get(), O.amax(xp, (0, 2)), 'amax padded')


@pytest.mark.parametrize('length', [10, 64, 100, 1000, 4096, 70000])
def test_argmax_ties_and_nans_bit_exact(length):
    """Rows full of ties and NaNs: the index must be the one the native backend's pairwise tree selects."""
    import chainer_amd as chx
    rng = np.random.default_rng(length)
    for trial in range(6):
        x = rng.integers(0, 4, (5, length)).astype('float32')
        if trial >= 2:
            x[rng.random((5, length)) < (0.02 if trial < 4 else 0.5)] = np.nan
        if trial == 5:
            x[:, 0] = np.nan
        X = chx.array(x)
        assert_exact(chx.argmax(X, 1).get(), O.argmax(x, 1), 'argmax rows t=%d' % trial)
        assert_exact(chx.amax(X, 1).get(), O.amax(x, 1), 'amax rows t=%d' % trial)
        xt = np.ascontiguousarray(x.T)
        assert_exact(chx.argmax(chx.array(xt), 0).get(), O.argmax(xt, 0), 'argmax columns t=%d' % trial)
    xz = np.array([[-0.0, 0.0, 0.0, -0.0]], 'float32')
    assert_exact(chx.argmax(chx.array(xz), 1).get(), O.argmax(xz, 1), 'signed zeros')


@pytest.mark.parametrize('dt', ['float16', 'float32', 'float64'])
def test_long_rows_with_few_nans_infinities_and_signed_zeros(dt):
    """The row kernel folds a wave's elements with a shorter comparison when none of them is NaN and with the full rule
    otherwise: rows in which only a few waves hold a NaN take both routes and must still give the native backend's answer
    bit for bit -- the index, which NaN-free maximum, and the sign of a zero maximum (the first of equal values wins)."""
    import chainer_amd as chx
    rng = np.random.default_rng(17)
    rows, length = 12, 9000
    x = rng.integers(-3, 1, (rows, length)).astype(dt)      # maximum 0, many ties
    x[x == 0] = np.where(rng.random(int((x == 0).sum())) < 0.5, 0.0, -0.0).astype(dt)  # zeros of both signs
    x[1, 5000] = np.nan                      # one NaN, one wave
    x[2, [17, 4100, 8999]] = np.nan          # the last one among the leftover groups
    x[3, 0] = np.nan                         # a leading NaN is never replaced
    x[4, 100] = np.inf
    x[4, 101] = -np.inf                      # inf - inf: the probe says NaN although there is none
    x[5, 2000:2300] = np.inf
    x[6, :] = -np.inf
    x[7, 1024:2048] = np.nan                 # a whole iteration of NaNs
    x[8, :] = np.where(rng.random(length) < 0.5, 0.0, -0.0).astype(dt)
    X = chx.array(x)
    for name in ('amax', 'amin', 'argmax', 'argmin'):
        assert_exact(getattr(chx, name)(X, 1).get(), getattr(O, name)(x, 1), '%s %s' % (name, dt))
    flat = chx.array(x.reshape(-1))           # one row split over several blocks
    for name in ('amax', 'amin', 'argmax', 'argmin'):
        assert_exact(getattr(chx, name)(flat, 0).get(), getattr(O, name)(x.reshape(-1), 0), '%s flat %s' % (name, dt))


@pytest.mark.parametrize('dt,tol', [('float32', 1e-5), ('float64', 1e-12), ('float16', 2e-2)])
def test_log_softmax_mean_softmax(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(1)
    x = rng.standard_normal((37, 1000)).astype(dt)
    X = chx.array(x)
    assert_close(chx.log_softmax(X, 1).get(), O.log_softmax(x, 1), tol, 'log_softmax')
    assert_close(chx.mean(X, 1).get(), O.mean(x, 1), tol, 'mean')
    sm = chx.softmax(X, 1).get().astype(np.float64)
    assert np.abs(sm.sum(1) - 1).max() < (2e-2 if dt == 'float16' else 1e-5)
    xi = rng.integers(-5, 5, (6, 7)).astype('int32')
    assert_close(chx.mean(chx.array(xi), 0).get(), O.mean(xi, 0), 1e-6, 'mean of ints is float32')


def test_softmax_cross_entropy():
    import chainer_amd as chx
    rng = np.random.default_rng(2)
    t = rng.integers(0, 10, 100).astype('int32')
    y = rng.standard_normal((100, 10)).astype('float32')
    assert_close(chx.softmax_cross_entropy(chx.array(y), chx.array(t)).get(), O.softmax_cross_entropy(y, t), 1e-5)


@pytest.mark.parametrize('shape', [(4096, 4096), (64, 1048576)])
def test_sweep_shapes_full_size(shape):
    """The elementwise/reduction sweep at its real sizes: argmax/amax bit-exact, sum bit-exact, log_softmax 1e-5,
    plus the size-independent properties (rows of exp(log_softmax) sum to 1; argmax indexes the max)."""
    import chainer_amd as chx
    rng = np.random.default_rng(3)
    x = rng.standard_normal(shape).astype('float32')
    X = chx.array(x)
    am = chx.argmax(X, 1).get()
    assert_exact(am, O.argmax(x, 1), 'argmax')
    assert_exact(chx.amax(X, 1).get(), O.amax(x, 1), 'amax')
    assert np.array_equal(x[np.arange(shape[0]), am], x.max(1))
    assert_exact(chx.sum(X, 1).get(), O.sum(x, 1), 'sum')
    ls = chx.log_softmax(X, 1)
    assert_close(ls.get(), O.log_softmax(x, 1), 1e-5, 'log_softmax')
    rows = chx.sum(chx.exp(ls), 1).get()
    assert np.abs(rows - 1).max() < 1e-4
    assert_exact(chx.sum(X, 0).get(), O.sum(x, 0), 'column sum')


def test_reduction_errors_and_empty():
    import chainer_amd as chx
    X = chx.array(np.zeros((2, 3), np.float32))
    with pytest.raises(chx.DimensionError):
        chx.sum(X, 2)
    with pytest.raises(chx.DimensionError):
        chx.argmax(X, -3)
    with pytest.raises(chx.DimensionError):
        chx.argmax(chx.zeros((2, 0, 3), 'float32'), 1)  # "cannot compute the argmax of an empty array" (routines/sorting.cc)
    assert chx.sum(chx.zeros((2, 0, 3), 'float32'), 1).get().tolist() == [[0, 0, 0], [0, 0, 0]]
    assert chx.argmax(chx.zeros((2, 0, 3), 'float32'), 2).get().shape == (2, 0)


@pytest.mark.parametrize('dt', ['float32', 'float16', 'int32', 'float64'])
def test_reduce_over_batch_and_plane_of_nchw(dt):
    """Axes (0, 2, 3) of a dense NCHW array: runs of H*W elements at a constant pitch per channel (batch-norm statistics, bias
    gradients).  Same pairwise tree over the flattened (n, h, w) sequence as the native backend, so sums stay bit-exact."""
    import chainer_amd as chx
    rng = np.random.default_rng(77)
    for shape in [(8, 6, 12, 12), (32, 16, 14, 14), (3, 5, 7, 8), (2, 4, 6, 6), (5, 3, 2, 128), (4, 7, 9, 9)]:
        if np.dtype(dt).kind == 'f':
            x = rng.standard_normal(shape).astype(dt)
        else:
            x = rng.integers(-100, 100, shape).astype(dt)
        X = chx.array(x)
        what = '%s %r' % (dt, shape)
        assert_exact(chx.sum(X, (0, 2, 3)).get(), O.sum(x, (0, 2, 3)), 'sum ' + what)
        assert_exact(chx.sum(X, (0, 2, 3), True).get(), O.sum(x, (0, 2, 3), True), 'sum keepdims ' + what)
        assert_exact(chx.amax(X, (0, 2, 3)).get(), O.amax(x, (0, 2, 3)), 'amax ' + what)
        assert_exact(chx.amin(X, (0, 2, 3)).get(), O.amin(x, (0, 2, 3)), 'amin ' + what)
        # a sliced batch axis keeps the pitch constant; a sliced plane breaks the runs (generic path)
        assert_exact(chx.sum(X[::2], (0, 2, 3)).get(), O.sum(x[::2], (0, 2, 3)), 'sum of every second image ' + what)
        assert_exact(chx.sum(X[:, :, ::2], (0, 2, 3)).get(), O.sum(x[:, :, ::2], (0, 2, 3)), 'sum of a strided plane ' + what)
    big = rng.standard_normal((16, 8, 56, 56)).astype(dt) if np.dtype(dt).kind == 'f' else rng.integers(-100, 100, (16, 8, 56, 56)).astype(dt)
    assert_exact(chx.sum(chx.array(big), (0, 2, 3)).get(), O.sum(big, (0, 2, 3)), 'rows split over several workgroups')


@pytest.mark.parametrize('dt', ['float32', 'float16', 'int32', 'float64', 'bool'])
def test_reduce_over_a_long_strided_axis(dt):
    """A long reduced axis that is not the contiguous one (sums over the batch axis, bias gradients of a linear layer): the
    sequence is cut into aligned slices that run in parallel and are merged through the native backend's binary counter, so every
    result stays bit-identical to the sequential tree -- including the tie and NaN choices of ArgMax / ArgMin."""
    import chainer_amd as chx
    rng = np.random.default_rng(91)
    cases = [((4096, 512), 0), ((100003, 64), 0), ((5000, 33), 0), ((513, 7), 0), ((1027, 300), 0), ((640, 3), 0), ((20001, 3, 5), 0),
             ((4, 9002, 6), 1), ((2049, 1), 0), ((70000, 2), 0)]
    for shape, axis in cases:
        if dt == 'bool':
            x = rng.random(shape) > 0.5
        elif np.dtype(dt).kind == 'f':
            x = rng.integers(0, 6, shape).astype(dt) if shape[0] == 5000 else rng.standard_normal(shape).astype(dt)
            if shape[0] == 1027:
                x[rng.random(shape) < 0.01] = np.nan
        else:
            x = rng.integers(-100, 100, shape).astype(dt)
        X = chx.array(x)
        what = '%s %r axis=%d' % (dt, shape, axis)
        assert_exact(chx.sum(X, axis).get(), O.sum(x, axis), 'sum ' + what)
        assert_exact(chx.sum(X, axis, True).get(), O.sum(x, axis, True), 'sum keepdims ' + what)
        assert_exact(chx.amax(X, axis).get(), O.amax(x, axis), 'amax ' + what)
        assert_exact(chx.amin(X, axis).get(), O.amin(x, axis), 'amin ' + what)
        assert_exact(chx.argmax(X, axis).get(), O.argmax(x, axis), 'argmax ' + what)
        assert_exact(chx.argmin(X, axis).get(), O.argmin(x, axis), 'argmin ' + what)
        if dt == 'bool':
            assert_exact(chx.all(X, axis).get(), O.all(x, axis), 'all ' + what)
            assert_exact(chx.any(X, axis).get(), O.any(x, axis), 'any ' + what)
    if dt != 'bool':  # a transposed view: the reduced axis is the contiguous one of the base array's other axis
        x = rng.standard_normal((48, 3000)).astype(dt) if np.dtype(dt).kind == 'f' else rng.integers(-100, 100, (48, 3000)).astype(dt)
        X = chx.array(x)
        assert_exact(chx.sum(X[:, ::3].T, 1).get(), O.sum(x[:, ::3].T, 1), 'sum over the strided axis of a view')
        assert_exact(chx.sum(X[:, ::3], 1).get(), O.sum(x[:, ::3], 1), 'sum over a stepped axis')

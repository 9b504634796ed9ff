"""Elementwise kernels (arithmetic, math, select, compare, copy/astype, fill, arange) against the CPU oracle.

Bar: bit-exact for everything that is a single IEEE operation or a copy (all nine dtypes, any strides); exp/log/tanh
are libm calls in the reference and are held to the float tolerance of the contract (1e-5 fp32, 2e-2 fp16)."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, padded, upload_view, channels_last

pytestmark = pytest.mark.gpu

ALL = ['bool', 'int8', 'int16', 'int32', 'int64', 'uint8', 'float16', 'float32', 'float64']
NUMERIC = ALL[1:]
FLOATS = ['float16', 'float32', 'float64']


def rand(rng, shape, dt):
    if dt == 'bool':
        return rng.random(shape) > 0.5
    if np.dtype(dt).kind == 'f':
        return (rng.standard_normal(shape) * 10).astype(dt)
    return rng.integers(0 if dt == 'uint8' else -100, 100, shape).astype(dt)


@pytest.mark.parametrize('dt', ALL)
def test_binary_arithmetic_all_layouts(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(0)
    x, y = rand(rng, (37, 53), dt), rand(rng, (37, 53), dt)
    b = rand(rng, (53,), dt)
    X, Y, B = chx.array(x), chx.array(y), chx.array(b)
    assert_exact((X + Y).get(), O.add(x, y), 'add')
    assert_exact((X * Y).get(), O.multiply(x, y), 'multiply')
    assert_exact((X + B).get(), O.add(x, np.broadcast_to(b, x.shape)), 'add broadcast (stride 0)')
    assert_exact((X * B).get(), O.multiply(x, np.broadcast_to(b, x.shape)), 'multiply broadcast')
    assert_exact((X.T + Y.T).get(), O.add(x.T, y.T), 'transposed views')
    assert_exact((X[3:30:2, 1:50:3] + Y[3:30:2, 1:50:3]).get(), O.add(x[3:30:2, 1:50:3], y[3:30:2, 1:50:3]), 'sliced views')
    assert_exact((X[::-1, ::-2] + Y[::-1, ::-2]).get(), O.add(x[::-1, ::-2], y[::-1, ::-2]), 'negative strides')
    if dt != 'bool':
        assert_exact((X - Y).get(), O.subtract(x, y), 'subtract')
        s = 3 if np.dtype(dt).kind != 'f' else 2.5
        sv = np.asarray(s).astype(dt)
        assert_exact((X + s).get(), O.add(x, sv), 'add scalar')
        assert_exact((X - s).get(), O.subtract(x, sv), 'subtract scalar')
        assert_exact((X * s).get(), O.multiply(x, sv), 'multiply scalar')
        assert_exact(chx.maximum(X, 0).get(), O.relu(x), 'relu')
    # in-place forms alias out with x1
    Z = X.copy()
    Z += Y
    assert_exact(Z.get(), O.add(x, y), 'iadd')
    # padded (non-contiguous in every axis) operands like the reference's WithPadding(1)
    xp, yp = padded((4, 3, 5), rand(rng, (4, 3, 5), dt), 1, dt), padded((4, 3, 5), rand(rng, (4, 3, 5), dt), 2, dt)
    assert_exact((upload_view(chx, xp) + upload_view(chx, yp)).get(), O.add(xp, yp), 'padded')


@pytest.mark.parametrize('dt', FLOATS)
def test_divide_and_math(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(1)
    x = rng.standard_normal((64, 1000)).astype(dt)
    X = chx.array(x)
    three = np.asarray(3, dt)
    with np.errstate(all='ignore'):
        assert_exact((X / (X + 3)).get(), O.divide(x, O.add(x, three)), 'divide')
        assert_exact((X / 3).get(), O.divide(x, three), 'divide scalar')
        assert_exact((3 / X).get(), O.divide(three, x), 'scalar / array')
        assert_exact(chx.sqrt(X).get(), O.sqrt(x), 'sqrt')
        tol = {'float16': 2e-3, 'float32': 1e-6, 'float64': 1e-14}[dt]
        for name in ('exp', 'tanh', 'log', 'sigmoid'):
            assert_close(getattr(chx, name)(X).get(), getattr(O, name)(x), tol, name)
    # strided (gate-like) views: every 4th column
    assert_close(chx.tanh(X[:, 1::4]).get(), O.tanh(x[:, 1::4]), tol, 'tanh strided')


def test_math_special_values():
    import chainer_amd as chx
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 88.8, -104.0, 1e-40, 710.0], np.float32)
    with np.errstate(all='ignore'):
        for name in ('exp', 'tanh', 'log', 'sqrt'):
            got, ref = getattr(chx, name)(chx.array(x)).get(), getattr(O, name)(x)
            assert np.array_equal(np.isnan(got), np.isnan(ref)), name
            assert np.array_equal(np.isinf(got), np.isinf(ref)), name
            fin = np.isfinite(ref)
            assert np.allclose(got[fin], ref[fin], rtol=1e-5, atol=1e-44), name
    r = chx.maximum(chx.array(x), 0).get()
    assert np.isnan(r[4]) and r[3] == 0 and r[2] == np.inf  # NaN < 0 is false: NaN passes through ReLU


@pytest.mark.parametrize('src', ALL)
def test_astype_all_pairs(src):
    import chainer_amd as chx
    rng = np.random.default_rng(2)
    x = rand(rng, (19, 21), src)
    if np.dtype(src).kind == 'f':
        x = np.abs(x)  # negative float -> unsigned is undefined behaviour in C++ as well
    X = chx.array(x)
    for dst in ALL:
        assert_exact(X.astype(dst).get(), O.astype(x, dst), '%s -> %s' % (src, dst))
        assert_exact(X.T[::2].astype(dst).get(), O.astype(x.T[::2], dst), '%s -> %s strided' % (src, dst))


def test_float16_rounding_on_store_exhaustive():
    """float32 -> float16 casts of values around every half and every midpoint: round-to-nearest-even (CX/float16.cc:27-89)."""
    import chainer_amd as chx
    h = np.arange(1 << 16, dtype=np.uint16).view(np.float16)
    f = h.astype(np.float32)
    f = f[np.isfinite(f)]
    mids = ((f[:-1].astype(np.float64) + np.roll(f, -1)[:-1].astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([f, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)), np.array([65519.9, 65520.0, 1e-8], np.float32)])
    got = chx.array(x).astype('float16').get()
    with np.errstate(all='ignore'):
        assert_exact(got, x.astype(np.float16))
    # half -> float is exact; NaNs compare as NaNs (the hardware conversion quiets signalling NaN payloads)
    assert_exact(chx.array(h).astype('float32').get(), h.astype(np.float32))


def test_compare_fill_arange():
    import chainer_amd as chx
    a = np.arange(6, dtype='int32')
    assert_exact((chx.array(a)[:, None] == chx.arange(4, dtype='int32')).get(), a[:, None] == np.arange(4, dtype='int32'))
    x = np.array([1.0, np.nan, 3.0], np.float32)
    y = np.array([1.0, np.nan, 2.0], np.float32)
    X, Y = chx.array(x), chx.array(y)
    assert (X == Y).get().tolist() == [True, False, False] and (X != Y).get().tolist() == [False, True, True]
    assert (X > Y).get().tolist() == [False, False, True] and (X >= Y).get().tolist() == [True, False, True]
    assert_exact(chx.arange(10, dtype='int32').get(), np.arange(10, dtype='int32'))
    assert_exact(chx.arange(0, 5, 0.5, dtype='float32').get(), np.arange(0, 5, 0.5, dtype='float32'))
    for dt in ALL:
        z = chx.full((3, 5), 1, dt)
        assert_exact(z.get(), np.full((3, 5), 1, dt))
        v = chx.zeros((4, 6), dt)
        v[1:3, ::2].fill(1)  # non-contiguous fill (array_test.cc:393-441)
        ref = np.zeros((4, 6), dt)
        ref[1:3, ::2] = 1
        assert_exact(v.get(), ref)
    assert chx.zeros((0, 3), 'float32').get().shape == (0, 3)  # zero-sized arrays are legal everywhere
    assert (chx.zeros((0, 3), 'float32') + chx.zeros((0, 3), 'float32')).shape == (0, 3)


def test_channels_last_views_and_large_shapes():
    import chainer_amd as chx
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 8, 5, 6)).astype('float16')
    X = channels_last(chx, x)
    assert_exact((X + X).get(), O.add(x, x), 'nhwc + nhwc')
    assert_exact((X + chx.array(x)).get(), O.add(x, x), 'nhwc + nchw')
    assert_exact(chx.maximum(X, 0).get(), O.relu(x), 'relu nhwc')
    # the sweep's shapes at full size: x + b, x * b (b broadcast over rows), relu -- bit-exact
    for shape in ((4096, 4096), (64, 1048576)):
        x = rng.standard_normal(shape).astype('float32')
        b = rng.standard_normal(shape[1]).astype('float32')
        X, B = chx.array(x), chx.array(b)
        assert_exact((X + B).get(), x + b, 'x+b %s' % (shape,))
        assert_exact((X * B).get(), x * b, 'x*b %s' % (shape,))
        with np.errstate(all='ignore'):
            assert_close(chx.exp(X).get(), np.exp(x), 1e-6, 'exp %s' % (shape,))
            assert_close(chx.tanh(X).get(), np.tanh(x), 1e-6, 'tanh %s' % (shape,))


def test_error_paths():
    import chainer_amd as chx
    X = chx.array(np.zeros((3, 4), np.float32))
    with pytest.raises(chx.DimensionError):
        X + chx.array(np.zeros((3, 5), np.float32))
    with pytest.raises(chx.ChainerxError):
        chx.subtract(chx.array(np.zeros(3, bool)), chx.array(np.zeros(3, bool)))  # bool subtract is rejected like numpy/ChainerX

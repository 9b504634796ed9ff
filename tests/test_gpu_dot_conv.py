"""Dot / Linear / Conv forward (MFMA implicit GEMM) against the CPU oracle: 1e-5 relative for float32, 2e-2 for float16
(products of the stored values, float32 accumulation, one rounding), 1e-12 for float64."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, channels_last, padded, upload_view
from test_oracle_pins import CONV_GRID

pytestmark = pytest.mark.gpu

DT = [('float32', 1e-5), ('float16', 2e-2), ('float64', 1e-12)]

CONV_CASES = [
    # N,C,H,W,K,R,S,stride,pad,cover_all
    (2, 3, 9, 8, 4, 3, 3, (2, 1), (1, 2), False),
    (2, 16, 8, 8, 32, 3, 3, 1, 1, False),
    (3, 64, 7, 7, 64, 1, 1, 1, 0, False),
    (2, 64, 14, 14, 256, 1, 1, 2, 0, False),
    (2, 32, 10, 10, 24, 3, 3, 2, 1, True),
    (1, 3, 32, 32, 64, 7, 7, 2, 3, False),
    (2, 8, 5, 5, 130, 3, 3, 1, 1, False),
    (1, 24, 6, 6, 70, 1, 1, 1, 0, False),
    (4, 128, 9, 9, 128, 3, 3, 1, 1, False),
    (2, 20, 6, 7, 9, 2, 3, (1, 2), (0, 1), True),
    (2, 3, 64, 64, 64, 7, 7, 2, 3, False),   # ImageNet stem geometry (dedicated float16 kernel)
    (1, 3, 30, 48, 64, 7, 7, 2, 3, False),   # same with an odd number of output rows
    # 1x1 tile shapes of the float16 NCHW kernel: 128x128 tiles with pixel pairs / single pixels, 128x256 and 64x256 tiles
    (2, 64, 8, 8, 128, 1, 1, 1, 0, False),
    (3, 32, 7, 7, 128, 1, 1, 1, 0, False),
    (2, 32, 8, 8, 256, 1, 1, 1, 0, False),
    (16, 32, 46, 46, 512, 1, 1, 2, 0, False),
    (2, 64, 7, 7, 320, 1, 1, 1, 0, False),
    # at most one tile per compute unit and an even number (>= 4) of channel chunks: two wave groups split the reduction
    (2, 256, 7, 7, 512, 1, 1, 1, 0, False),
    (2, 128, 14, 14, 128, 1, 1, 1, 0, False),
    (3, 128, 7, 7, 128, 1, 1, 1, 0, False),
    (2, 64, 7, 7, 128, 3, 3, 1, 1, False),
    (3, 64, 14, 14, 64, 3, 3, 1, 1, False),
    (1, 64, 56, 56, 64, 3, 3, 1, 1, False),
    (5, 96, 7, 7, 70, 3, 3, 1, 1, False),
]


@pytest.mark.parametrize('dt,tol', DT)
def test_conv_layouts_and_shapes(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(0)
    for (N, C, H, W, K, R, S, st, pd, cv) in CONV_CASES:
        x = rng.standard_normal((N, C, H, W)).astype(dt)
        w = (rng.standard_normal((K, C, R, S)) / np.sqrt(C * R * S)).astype(dt)
        b = rng.standard_normal(K).astype(dt)
        ref = O.conv(x, w, b, st, pd, cv)
        what = '%s %s' % (dt, (N, C, H, W, K, R, S, st, pd, cv))
        for lay, X in (('nchw', chx.array(x)), ('nhwc', channels_last(chx, x))):
            y = chx.conv(X, chx.array(w), chx.array(b), st, pd, cv)
            assert y.shape == ref.shape and y.dtype == ref.dtype
            assert_close(y.get(), ref, tol, 'conv %s %s' % (lay, what))
        y = chx.conv(channels_last(chx, x), chx.array(w), None, st, pd, cv)
        assert_close(y.get(), O.conv(x, w, None, st, pd, cv), tol, 'conv without bias ' + what)


@pytest.mark.parametrize('xs,ws,bias,stride,pad', CONV_GRID)
@pytest.mark.parametrize('cover_all', [False, True])
def test_conv_reference_grid(xs, ws, bias, stride, pad, cover_all):
    """The 2-D rows of the reference's own parameter grid (test_connection.py:183-203), padded (non-contiguous) x."""
    import chainer_amd as chx
    rng = np.random.default_rng(1)
    for dt, tol in DT:
        x = padded(xs, rng.standard_normal(xs), 1, dt)
        w = (rng.standard_normal(ws) / np.sqrt(np.prod(ws[1:]))).astype(dt)
        b = rng.standard_normal(ws[0]).astype(dt) if bias else None
        y = chx.conv(upload_view(chx, x), chx.array(w), chx.array(b) if bias else None, stride, pad, cover_all)
        assert_close(y.get(), O.conv(x, w, b, stride, pad, cover_all), tol)


@pytest.mark.parametrize('dt,tol', DT)
def test_dot_and_linear(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(2)
    for (m, k, n) in [(100, 784, 1000), (7, 33, 5), (128, 650, 2600), (64, 64, 64), (1, 1, 1), (130, 100, 70), (3, 2000, 3)]:
        a = rng.standard_normal((m, k)).astype(dt)
        b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(dt)
        ref = O.dot(a, b)
        what = '%s %s' % (dt, (m, k, n))
        assert_close(chx.dot(chx.array(a), chx.array(b)).get(), ref, tol, 'dot ' + what)
        bt = chx.array(np.ascontiguousarray(b.T)).T  # the W^T view Linear passes (strides (item, item*K))
        assert_close(chx.dot(chx.array(a), bt).get(), ref, tol, 'dot with transposed-view b ' + what)
        at = chx.array(np.ascontiguousarray(a.T)).T
        assert_close(chx.dot(at, bt).get(), ref, tol, 'dot with both operands transposed views ' + what)
        bias = rng.standard_normal(n).astype(dt)
        wt = np.ascontiguousarray(b.T)
        assert_close(chx.linear(chx.array(a), chx.array(wt), chx.array(bias)).get(), O.linear(a, wt, bias), tol, 'linear ' + what)
    ap = padded((5, 9), rng.standard_normal((5, 9)), 1, dt)
    bp = padded((9, 4), rng.standard_normal((9, 4)), 2, dt)
    assert_close(chx.dot(upload_view(chx, ap), upload_view(chx, bp)).get(), O.dot(ap, bp), tol, 'padded operands')


def test_dot_integer_valued_is_exact():
    import chainer_amd as chx
    rng = np.random.default_rng(3)
    for dt in ('float32', 'float16', 'float64'):
        a = rng.integers(-3, 4, (70, 90)).astype(dt)
        b = rng.integers(-3, 4, (90, 50)).astype(dt)
        got = chx.dot(chx.array(a), chx.array(b)).get()
        assert np.array_equal(got.astype(np.int64), a.astype(np.int64) @ b.astype(np.int64))


INT_DTYPES = ('int8', 'uint8', 'int16', 'int32', 'int64')


def test_dot_and_linear_of_integers_and_bool():
    """The native backend multiplies every dtype (dot.cc:177-227); integer sums are arithmetic modulo 2^bits, so the results
    are equal bit for bit over the full value range, whatever the layout of the operands."""
    import chainer_amd as chx
    rng = np.random.default_rng(31)
    for dt in INT_DTYPES:
        info = np.iinfo(dt)
        for (m, k, n) in [(7, 33, 5), (64, 64, 64), (130, 100, 70), (1, 1, 1), (3, 2000, 3), (100, 17, 129)]:
            a = rng.integers(info.min, info.max, (m, k), dtype=dt, endpoint=True)
            b = rng.integers(info.min, info.max, (k, n), dtype=dt, endpoint=True)
            ref = O.dot(a, b)
            what = '%s %s' % (dt, (m, k, n))
            got = chx.dot(chx.array(a), chx.array(b))
            assert got.dtype == ref.dtype and np.array_equal(got.get(), ref), what
            at = chx.array(np.ascontiguousarray(a.T)).T
            bt = chx.array(np.ascontiguousarray(b.T)).T
            assert np.array_equal(chx.dot(at, bt).get(), ref), 'transposed views ' + what
            bias = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
            wt = np.ascontiguousarray(b.T)
            assert np.array_equal(chx.linear(chx.array(a), chx.array(wt), chx.array(bias)).get(), O.linear(a, wt, bias)), 'linear ' + what
        ap = padded((5, 9), rng.integers(-100, 100, (5, 9)), 1, dt)
        bp = padded((9, 4), rng.integers(-100, 100, (9, 4)), 2, dt)
        assert np.array_equal(chx.dot(upload_view(chx, ap), upload_view(chx, bp)).get(), O.dot(np.ascontiguousarray(ap), np.ascontiguousarray(bp)))
    a = rng.integers(0, 3, (70, 90)) == 0
    b = rng.integers(0, 20, (90, 50)) == 0
    got = chx.dot(chx.array(a), chx.array(b))
    assert got.dtype == np.bool_ and np.array_equal(got.get(), O.dot(a, b))
    # mixed operand dtypes are cast to the result dtype first (dot.cc:177-178)
    a8 = rng.integers(-128, 127, (9, 11), dtype='int8')
    b32 = rng.integers(-2 ** 31, 2 ** 31 - 1, (11, 6), dtype='int32')
    assert np.array_equal(chx.dot(chx.array(a8), chx.array(b32)).get(), O.dot(a8.astype('int32'), b32))
    z = chx.dot(chx.zeros((3, 0), 'int32'), chx.zeros((0, 4), 'int32'))
    assert z.dtype == np.int32 and z.shape == (3, 4) and not z.get().any()


def test_conv_of_integers_over_any_number_of_axes():
    """Integer convolutions (the native backend's Im2Col + TensorDot takes every dtype): equal to the oracle bit for bit, values
    large enough to wrap, 0 to 3 spatial axes, dense and permuted input."""
    import chainer_amd as chx
    rng = np.random.default_rng(32)
    cases = [((2, 3), (4, 3), 1, 0), ((2, 3, 9), (4, 3, 3), 2, 1), ((2, 3, 7, 6), (5, 3, 3, 2), (2, 1), (1, 0)),
             ((3, 16, 8, 8), (32, 16, 3, 3), 1, 1), ((2, 2, 5, 4, 6), (3, 2, 2, 3, 2), (1, 2, 1), (1, 0, 1))]
    for dt in INT_DTYPES + ('bool',):
        for xs, ws, stride, pad in cases:
            if dt == 'bool':
                x, w, b = (rng.integers(0, 4, xs) == 0), (rng.integers(0, 4, ws) == 0), (rng.integers(0, 4, ws[0]) == 0)
            else:
                info = np.iinfo(dt)
                lo, hi = max(info.min, -2 ** 20), min(info.max, 2 ** 20)
                x, w, b = (rng.integers(lo, hi, s).astype(dt) for s in (xs, ws, ws[0]))
            for cv in (False, True):
                for bias in (None, b):
                    ref = O.conv_nd(x, w, bias, stride, pad, cv)
                    got = chx.conv(chx.array(x), chx.array(w), chx.array(bias) if bias is not None else None, stride, pad, cv)
                    assert got.dtype == ref.dtype and got.shape == ref.shape, (dt, xs, ws)
                    assert np.array_equal(got.get(), ref), (dt, xs, ws, stride, pad, cv, bias is not None)
            if len(xs) == 4:
                got = chx.conv(channels_last(chx, x), chx.array(w), chx.array(b), stride, pad)
                assert np.array_equal(got.get(), O.conv_nd(x, w, b, stride, pad)), ('permuted', dt, xs)


def test_dot_conv_edge_cases_and_errors():
    import chainer_amd as chx
    z = chx.dot(chx.zeros((3, 0), 'float32'), chx.zeros((0, 4), 'float32')).get()
    assert z.shape == (3, 4) and not z.any()  # k == 0 -> zeros (CX/routines/linalg.cc:59-61)
    assert chx.dot(chx.zeros((0, 5), 'float32'), chx.zeros((5, 4), 'float32')).shape == (0, 4)
    with pytest.raises(chx.DimensionError):
        chx.dot(chx.zeros((3, 4), 'float32'), chx.zeros((5, 4), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.conv(chx.zeros((1, 3, 4, 4), 'float32'), chx.zeros((2, 4, 3, 3), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.conv(chx.zeros((1, 3, 2, 2), 'float32'), chx.zeros((2, 3, 5, 5), 'float32'))  # output size not positive
    assert chx.conv(chx.zeros((0, 3, 4, 4), 'float32'), chx.zeros((2, 3, 3, 3), 'float32')).shape == (0, 2, 2, 2)


def test_conv_linearity_at_resnet_layer_size():
    """Size-independent property at a real layer shape (fp16 [32,256,14,14] * [256,256,3,3]): conv(x, w1 + w2) matches
    conv(x, w1) + conv(x, w2) to rounding, and a delta filter reproduces the input."""
    import chainer_amd as chx
    rng = np.random.default_rng(4)
    x = rng.standard_normal((32, 256, 14, 14)).astype('float16')
    w1 = (rng.standard_normal((256, 256, 3, 3)) / 48).astype('float16')
    w2 = (rng.standard_normal((256, 256, 3, 3)) / 48).astype('float16')
    X = chx.array(x)
    y1 = chx.conv(X, chx.array(w1), None, 1, 1).get().astype(np.float64)
    y2 = chx.conv(X, chx.array(w2), None, 1, 1).get().astype(np.float64)
    w12 = (w1.astype(np.float32) + w2.astype(np.float32)).astype('float16')
    y12 = chx.conv(X, chx.array(w12), None, 1, 1).get().astype(np.float64)
    scale = np.abs(y1 + y2).max()
    assert np.abs(y12 - (y1 + y2)).max() / scale < 2e-2
    delta = np.zeros((256, 256, 3, 3), 'float16')
    delta[np.arange(256), np.arange(256), 1, 1] = 1
    assert np.array_equal(chx.conv(X, chx.array(delta), None, 1, 1).get(), x)


def test_pointwise_conv_with_more_tiles_than_resident_workgroups():
    """A 1x1 convolution whose tile count (1568 tiles of 128 x 128) exceeds what the device holds at once, so that every
    workgroup walks several tiles: against the oracle, with a bias, and an identity filter bank reproduces the input bit for bit
    (each output tile lands where it belongs)."""
    import chainer_amd as chx
    rng = np.random.default_rng(14)
    x = rng.standard_normal((32, 64, 56, 56)).astype('float16')
    w = (rng.standard_normal((256, 64, 1, 1)) / 8).astype('float16')
    b = rng.standard_normal(256).astype('float16')
    got = chx.conv(chx.array(x), chx.array(w), chx.array(b)).get()
    assert_close(got, O.conv(x, w, b), 2e-2, 'conv 1x1, 1568 tiles')
    eye = np.zeros((256, 64, 1, 1), 'float16')
    eye[np.arange(256), np.arange(256) % 64, 0, 0] = 1
    out = chx.conv(chx.array(x), chx.array(eye)).get()
    assert np.array_equal(out, np.tile(x, (1, 4, 1, 1)))


@pytest.mark.parametrize('dt,tol', DT)
def test_dot_operand_layouts_large(dt, tol):
    """Products large enough for the tiled MFMA kernel with every operand layout Dot accepts without a copy in the reference
    (native/native_device/dot.cc:51-77): row-major and transposed views on either side, odd reduction lengths, padded pitches."""
    import chainer_amd as chx
    rng = np.random.default_rng(9)
    for (m, k, n) in [(1200, 100, 1800), (1200, 101, 1800), (1500, 64, 1300)]:
        a = (rng.standard_normal((m, k)) / np.sqrt(k)).astype(dt)
        b = rng.standard_normal((k, n)).astype(dt)
        ref = O.dot(a, b)
        A_row, B_row = chx.array(a), chx.array(b)
        A_t = chx.array(np.ascontiguousarray(a.T)).T          # unit stride along m
        B_t = chx.array(np.ascontiguousarray(b.T)).T          # unit stride along k
        for la, A in (('a row-major', A_row), ('a transposed view', A_t)):
            for lb, B in (('b row-major', B_row), ('b transposed view', B_t)):
                assert_close(chx.dot(A, B).get(), ref, tol, 'dot %s %s, %s, %s' % (dt, (m, k, n), la, lb))
        # padded parents: pitches that are no multiple of the row length
        ap = padded((m, k), a, 1, dt)
        bp = padded((k, n), b, 1, dt)
        assert_close(chx.dot(upload_view(chx, ap), upload_view(chx, bp)).get(), ref, tol, 'dot of padded operands %r' % ((m, k, n),))


@pytest.mark.parametrize('N,C,H,K', [(8, 16, 56, 192), (16, 16, 28, 384), (32, 16, 14, 704), (64, 16, 7, 1344), (2, 32, 7, 128), (3, 16, 14, 64),
                                     (2, 16, 28, 64), (1, 16, 56, 64)])
def test_conv3x3_float16_tile_variants(N, C, H, K):
    """3x3 / stride 1 / pad 1 on dense float16 NCHW, from grids of several hundred 256-pixel tiles down to a single partial tile,
    for even (pixel pairs) and odd (single pixels) plane widths."""
    import chainer_amd as chx
    rng = np.random.default_rng(N * 100 + H)
    x = rng.standard_normal((N, C, H, H)).astype('float16')
    w = (rng.standard_normal((K, C, 3, 3)) / np.sqrt(C * 9)).astype('float16')
    b = rng.standard_normal(K).astype('float16')
    y = chx.conv(chx.array(x), chx.array(w), chx.array(b), 1, 1)
    assert_close(y.get(), O.conv(x, w, b, 1, 1, False), 2e-2, 'conv3x3 %r' % ((N, C, H, K),))


@pytest.mark.parametrize('dt,tol', [('float32', 1e-5), ('float16', 2e-2)])
def test_dot_long_reduction_few_tiles(dt, tol):
    """Few output tiles over a long reduction axis (the weight-gradient shape): slices of the reduction run as separate workgroups
    and are summed in float.  Operands as the callers hand them over: a row-major, b the transposed view of a row-major [N, K]."""
    import chainer_amd as chx
    rng = np.random.default_rng(12)
    for (m, k, n) in [(128, 8192, 256), (200, 5000, 130), (64, 16384, 64), (256, 4096, 576), (70, 6000, 300)]:
        a = rng.standard_normal((m, k)).astype(dt)
        bt = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(dt)
        ref = O.dot(a, np.ascontiguousarray(bt.T))
        got = chx.dot(chx.array(a), chx.array(bt).T)
        assert_close(got.get(), ref, tol, 'dot %s %r' % (dt, (m, k, n)))
        out_t = chx.dot(chx.array(bt), chx.array(a).T)  # the same product transposed: [n, m]
        assert_close(out_t.get(), ref.T.copy(), tol, 'dot transposed %s %r' % (dt, (m, k, n)))


@pytest.mark.parametrize('dt,tol', [('float32', 1e-5), ('float16', 2e-2)])
def test_dot_staged_operands_with_split_reduction(dt, tol):
    """128 to 256 output tiles over a reduction of 4096 or more with an operand that is not laid out along the reduction axis:
    the operand is staged in the workspace and the reduction is split as well, so the float partial sums must lie behind the
    staged copy, not on top of it.  Too large for the serial oracle loop: checked against the float64 product of the stored
    values (the oracle's own result lies within the same bound of it)."""
    import chainer_amd as chx
    rng = np.random.default_rng(21)
    for (m, k, n) in [(1536, 4096, 1536), (2048, 4096, 1024), (1536, 4100, 1300)]:
        a = rng.standard_normal((m, k)).astype(dt)
        b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(dt)
        ref = (a.astype(np.float64) @ b.astype(np.float64)).astype(dt)
        A_row, B_row = chx.array(a), chx.array(b)
        A_t = chx.array(np.ascontiguousarray(a.T)).T
        B_t = chx.array(np.ascontiguousarray(b.T)).T
        for la, A in (('a row-major', A_row), ('a transposed view', A_t)):
            for lb, B in (('b row-major', B_row), ('b transposed view', B_t)):
                assert_close(chx.dot(A, B).get(), ref, tol, 'dot %s %r, %s, %s' % (dt, (m, k, n), la, lb))


def test_dot_float16_256_tiles():
    """float16 products large enough for the 256 x 256 tile kernel (at least 192 such tiles, reduction a multiple of 32): exact on
    integer-valued data (float accumulation of small integers has no rounding), partial tiles on both edges, padded pitches, and
    every operand layout (row-major operands are staged into the layout the kernel reads).  Too large for the serial oracle
    loop: random data is checked against the float64 product of the stored values."""
    import chainer_amd as chx
    rng = np.random.default_rng(31)
    for (m, k, n) in [(4096, 96, 4096), (3600, 160, 3700), (2304, 1024, 6148)]:
        a = rng.integers(-3, 4, (m, k)).astype('float16')
        bt = rng.integers(-3, 4, (n, k)).astype('float16')
        ref = (a.astype(np.int64) @ bt.astype(np.int64).T)
        assert np.abs(ref).max() < 2048  # every result is a float16 value
        got = chx.dot(chx.array(a), chx.array(bt).T).get()
        assert np.array_equal(got.astype(np.int64), ref), 'integer-valued dot %r' % ((m, k, n),)
    m, k, n = 3840, 512, 4104
    a = rng.standard_normal((m, k)).astype('float16')
    b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype('float16')
    ref = (a.astype(np.float64) @ b.astype(np.float64)).astype('float16')
    A_row, B_row = chx.array(a), chx.array(b)
    A_t = chx.array(np.ascontiguousarray(a.T)).T
    B_t = chx.array(np.ascontiguousarray(b.T)).T
    for la, A in (('a row-major', A_row), ('a transposed view', A_t)):
        for lb, B in (('b row-major', B_row), ('b transposed view', B_t)):
            assert_close(chx.dot(A, B).get(), ref, 2e-2, 'dot %r, %s, %s' % ((m, k, n), la, lb))
    ap = padded((m, k), a, (8, 0), 'float16')        # row pitch k + 8 halves: 16-byte aligned rows
    btp = padded((n, k), np.ascontiguousarray(b.T), (24, 0), 'float16')
    got = chx.dot(upload_view(chx, ap), upload_view(chx, btp).T).get()
    assert_close(got, ref, 2e-2, 'dot of operands with padded pitches')


def test_conv1x1_float16_lds_direct_ring():
    """1x1 / stride 1 float16 layers on the kernel that loads its operands straight into LDS (route 3; four-wave workgroups on
    256-pixel x 128-channel tiles, two to a compute unit): planes whose pixel count is a multiple of 8 and of 4
    only (the last 16-byte piece of a plane is then half empty), workgroups that walk more than one tile, partial channel tiles,
    bias.  Integer-valued data: float accumulation has no rounding, so results are exact and the rounding of the bias sum is the
    only one.  Too large for the serial oracle loop: the reference is the same sum of products in float64."""
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(41)
    cases = [(128, 64, 28, 256, True), (128, 64, 14, 1024, True), (96, 96, 14, 1320, False), (256, 32, 28, 128, True), (340, 160, 20, 100, True),
             (128, 512, 28, 128, False), (1600, 64, 6, 300, True)]
    for (n, c, hw, k, with_bias) in cases:
        x = rng.integers(-3, 4, (n, c, hw, hw)).astype('float16')
        w = rng.integers(-2, 3, (k, c, 1, 1)).astype('float16')
        b = rng.integers(-8, 9, k).astype('float16') if with_bias else None
        X, W, B = chx.array(x), chx.array(w), (chx.array(b) if with_bias else None)
        assert routines.conv_route(X, W, B) == 3, 'expected the LDS-direct 1x1 kernel for %r' % ((n, c, hw, k),)
        got = chx.conv(X, W, B).get()
        ref = np.einsum('nchw,kc->nkhw', x.astype(np.float32), w[:, :, 0, 0].astype(np.float32))
        if with_bias:
            ref = ref + b.astype(np.float32)[None, :, None, None]
        assert np.abs(ref).max() <= 2048
        assert np.array_equal(got.astype(np.float32), ref), 'conv 1x1 %r' % ((n, c, hw, k),)
    # random data against the float64 sum of products
    n, c, hw, k = 128, 256, 14, 1024
    x = rng.standard_normal((n, c, hw, hw)).astype('float16')
    w = (rng.standard_normal((k, c, 1, 1)) / np.sqrt(c)).astype('float16')
    b = rng.standard_normal(k).astype('float16')
    X, W, B = chx.array(x), chx.array(w), chx.array(b)
    assert routines.conv_route(X, W, B) == 3
    got = chx.conv(X, W, B).get()
    ref = (np.einsum('nchw,kc->nkhw', x.astype(np.float64), w[:, :, 0, 0].astype(np.float64)) + b.astype(np.float64)[None, :, None, None]).astype('float16')
    assert_close(got, ref, 2e-2, 'conv 1x1 %r' % ((n, c, hw, k),))
    # the general kernels keep the shapes the plan leaves out
    small = chx.array(rng.standard_normal((2, 64, 14, 14)).astype('float16'))
    assert routines.conv_route(small, chx.array(w[:256, :64])) != 3


@pytest.mark.parametrize('cover_all', [False, True])
def test_conv_and_pooling_over_n_axes_reference_grid(cover_all):
    """The rows of the reference's grids that are not 2-D (test_connection.py:178-203: 0, 1 and 3 spatial axes; test_pooling.py:15-27:
    1, 3 and 4) and the 2-D ones through the same entry points, against the oracle's n-axis restatements; dense and padded
    (non-contiguous) inputs, with and without bias, both pad modes, NaN / inf in pooling windows, larger 3-D cases."""
    import chainer_amd as chx
    from test_oracle_pins import CONV_ND_GRID, POOL_ND_GRID
    rng = np.random.default_rng(17)
    conv_cases = CONV_ND_GRID + [((2, 8, 5, 9, 7), (6, 8, 3, 3, 3), 1, 1), ((3, 4, 6, 6, 6), (5, 4, 2, 3, 1), (2, 1, 2), (0, 1, 0)),
                                 ((4, 16, 40), (8, 16, 5), 2, 2), ((5, 32), (7, 32), 1, 0)]
    for dt, tol in DT:
        for xs, ws, stride, pad in conv_cases:
            x = rng.standard_normal(xs).astype(dt)
            w = (rng.standard_normal(ws) / np.sqrt(np.prod(ws[1:]))).astype(dt)
            b = rng.standard_normal(ws[0]).astype(dt)
            what = 'conv %s %r' % (dt, (xs, ws, stride, pad, cover_all))
            for bias in (None, b):
                ref = O.conv_nd(x, w, bias, stride, pad, cover_all)
                y = chx.conv(chx.array(x), chx.array(w), chx.array(bias) if bias is not None else None, stride, pad, cover_all)
                assert y.shape == ref.shape and y.dtype == ref.dtype, what
                assert_close(y.get(), ref, tol, what)
            if len(xs) > 2:
                xp = padded(xs, x, 1, dt)
                y = chx.conv(upload_view(chx, xp), chx.array(w), chx.array(b), stride, pad, cover_all)
                assert_close(y.get(), O.conv_nd(x, w, b, stride, pad, cover_all), tol, what + ' (padded x)')
        pool_cases = POOL_ND_GRID + [((2, 5, 6, 7, 8), (3, 2, 3), (2, 1, 2), (1, 0, 1)), ((3, 4, 33), (4,), 3, 1)]
        for xs, ks, stride, pad in pool_cases:
            x = rng.standard_normal(xs).astype(dt)
            what = 'pool %s %r' % (dt, (xs, ks, stride, pad, cover_all))
            got = chx.max_pool(chx.array(x), ks, stride, pad, cover_all).get()
            assert np.array_equal(got, O.max_pool_nd(x, ks, stride, pad, cover_all)), 'max_' + what
            xn = x.copy()
            xn.reshape(-1)[::7] = np.nan
            xn.reshape(-1)[3::11] = np.inf
            got = chx.max_pool(chx.array(xn), ks, stride, pad, cover_all).get()
            assert np.array_equal(got, O.max_pool_nd(xn, ks, stride, pad, cover_all), equal_nan=True), 'max_' + what + ' with NaN / inf'
            if not cover_all:
                for mode in ('zero', 'ignore'):
                    got, ref = chx.average_pool(chx.array(x), ks, stride, pad, mode).get(), O.average_pool_nd(x, ks, stride, pad, mode)
                    fin = np.isfinite(ref)
                    assert got.shape == ref.shape and np.array_equal(np.isnan(got), np.isnan(ref)), 'average_%s %s' % (what, mode)
                    assert_close(np.where(fin, got, 0), np.where(fin, ref, 0), tol * 2, 'average_%s %s' % (what, mode))
        xi = rng.integers(-50, 50, (2, 3, 4, 5, 6)).astype('int32')
        assert np.array_equal(chx.max_pool(chx.array(xi), (2, 2, 3), 2, 1, cover_all).get(), O.max_pool_nd(xi, (2, 2, 3), 2, 1, cover_all))
    with pytest.raises(chx.DimensionError):
        chx.conv(chx.zeros((1, 3, 4, 4, 4), 'float32'), chx.zeros((2, 4, 1, 1, 1), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.max_pool(chx.zeros((1, 3, 2, 2, 2), 'float32'), 3, 1, 0)

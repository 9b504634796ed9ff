"""hipcx_im2col / hipcx_col2im / hipcx_conv_transpose against the CPU oracle and against the kernel-by-kernel compositions.

Bar: im2col is a gather (bit-exact); col2im reproduces the native backend's chain of in-place strided additions, including the
rounding after every addition (bit-exact); conv_transpose within the float tolerance (its stride-1 route sums in another order)."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, channels_last, padded, upload_view

pytestmark = pytest.mark.gpu

# (x shape, kernel, stride, pad, cover_all)
WINDOWS = [((2, 3, 7, 9), (3, 3), (1, 1), (1, 1), False), ((2, 3, 7, 9), (3, 2), (2, 3), (0, 1), False),
           ((1, 5, 8, 8), (2, 2), (2, 2), (0, 0), False), ((2, 2, 9, 7), (3, 3), (2, 2), (1, 1), True),
           ((1, 1, 5, 5), (5, 5), (1, 1), (2, 2), False), ((3, 4, 6, 6), (1, 1), (2, 2), (0, 0), False),
           ((2, 2, 10, 11), (4, 3), (3, 2), (2, 1), True), ((1, 2, 4, 4), (3, 3), (1, 1), (3, 3), False)]


@pytest.mark.parametrize('dt', ['float32', 'float16', 'float64', 'int32', 'int8', 'bool'])
def test_im2col_matches_the_oracle_and_the_copy_chain(dt):
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(70)
    for shape, k, s, p, cv in WINDOWS:
        if dt == 'bool':
            x, pv = rng.random(shape) > 0.5, False
        elif np.dtype(dt).kind == 'f':
            x, pv = rng.standard_normal(shape).astype(dt), -np.inf
        else:
            x, pv = rng.integers(-100, 100, shape).astype(dt), -7
        ref = O._windows(x, k, s, p, cv, pv)
        what = '%s %r' % (dt, (shape, k, s, p, cv))
        assert_exact(routines.im2col(chx.array(x), k, s, p, cv, pv).get(), ref, 'im2col ' + what)
        assert_exact(routines.im2col(channels_last(chx, x), k, s, p, cv, pv).get(), ref, 'im2col of a channels-last x ' + what)
        routines.COMPOSE_IM2COL = True
        try:
            chain = routines.im2col(chx.array(x), k, s, p, cv, pv).get()
        finally:
            routines.COMPOSE_IM2COL = False
        assert_exact(chain, ref, 'im2col as a chain of strided copies ' + what)


@pytest.mark.parametrize('dt', ['float32', 'float16', 'float64', 'int32', 'int8'])
def test_col2im_carries_the_bits_of_the_in_place_add_chain(dt):
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(71)
    for shape, k, s, p, cv in WINDOWS:
        oh = O.conv_out_dim(shape[2], k[0], s[0], p[0], cv)
        ow = O.conv_out_dim(shape[3], k[1], s[1], p[1], cv)
        cshape = (shape[0], shape[1], k[0], k[1], oh, ow)
        if np.dtype(dt).kind == 'f':
            col = (rng.standard_normal(cshape) * 3).astype(dt)  # float16: sums of up to 25 terms round at every step
        else:
            col = rng.integers(-60, 60, cshape).astype(dt)       # int8 wraps
        ref = np.ascontiguousarray(O._col2im(col, s, p, shape[2:]))
        what = '%s %r' % (dt, (shape, k, s, p, cv))
        assert_exact(routines.col2im(chx.array(col), s, p, shape[2:]).get(), ref, 'col2im ' + what)
        # the layout ConvTranspose hands over: [C, kh, kw, N, h, w] memory seen as [N, C, kh, kw, h, w]
        colt = chx.array(np.ascontiguousarray(col.transpose(1, 2, 3, 0, 4, 5))).transpose((3, 0, 1, 2, 4, 5))
        assert_exact(routines.col2im(colt, s, p, shape[2:]).get(), ref, 'col2im of a transposed col ' + what)
        routines.COMPOSE_IM2COL = True
        try:
            chain = routines.col2im(chx.array(col), s, p, shape[2:]).get()
        finally:
            routines.COMPOSE_IM2COL = False
        assert_exact(chain, ref, 'col2im as a chain of strided additions ' + what)


def test_im2col_col2im_argument_checks():
    import chainer_amd as chx
    from chainer_amd import _lib, routines
    x = chx.array(np.zeros((1, 2, 5, 5), 'float32'))
    col = chx.ndarray.empty((1, 2, 3, 3, 4, 4), 'float32')  # 5 -> 3 window positions at stride 1 without padding, not 4
    with pytest.raises(chx.DimensionError):
        _lib.call('hipcx_im2col', x.desc(), routines._i64((1, 1)), routines._i64((0, 0)), 0, _lib.make_scalar(0), col.desc(), None)
    with pytest.raises(chx.DtypeError):
        _lib.call('hipcx_col2im', chx.ndarray.empty((1, 2, 3, 3, 3, 3), 'float16').desc(), routines._i64((1, 1)), routines._i64((0, 0)),
                  x.desc(), None)
    with pytest.raises(chx.DimensionError):
        _lib.call('hipcx_col2im', chx.ndarray.empty((1, 3, 3, 3, 3, 3), 'float32').desc(), routines._i64((1, 1)), routines._i64((0, 0)),
                  x.desc(), None)


# (N, C_in, H, W, C_out, kh, kw, stride, pad, out_size or None)
TRANSPOSE_CASES = [
    (2, 6, 5, 6, 4, 3, 3, 2, 1, None), (2, 6, 5, 6, 4, 3, 3, 2, 1, (10, 12)),      # the composition; a cover_all output size
    (1, 8, 4, 4, 8, 4, 4, 2, 1, None), (2, 3, 6, 5, 5, (2, 3), None, (3, 2), (0, 1), None),
    (2, 16, 7, 7, 8, 1, 1, 2, 0, None), (2, 16, 7, 7, 8, 1, 1, 2, 0, (14, 14)), (1, 4, 5, 5, 6, 1, 1, 3, 0, (13, 14)),  # scattered 1x1
    (2, 8, 9, 9, 12, 3, 3, 1, 1, None), (2, 8, 9, 9, 12, 5, 5, 1, 0, None), (4, 64, 14, 14, 32, 3, 3, 1, 1, None),  # flipped convolution
]


@pytest.mark.parametrize('dt,tol', [('float32', 1e-5), ('float16', 2e-2), ('float64', 1e-12)])
def test_conv_transpose_entry_against_oracle_and_routine_level_routing(dt, tol):
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(72)
    for case in TRANSPOSE_CASES:
        n, ci, h, wd, co, kh, kw, st, pd, out_size = case
        if kw is None:
            kh, kw = kh
        x = rng.standard_normal((n, ci, h, wd)).astype(dt)
        w = (rng.standard_normal((ci, co, kh, kw)) / np.sqrt(ci)).astype(dt)
        b = rng.standard_normal(co).astype(dt)
        what = '%s %r' % (dt, case)
        for bias, bd in ((None, None), (b, chx.array(b))):
            ref = O.conv_transpose(x, w, bias, st, pd, out_size)
            got = chx.conv_transpose(chx.array(x), chx.array(w), bd, st, pd, out_size)
            assert got.shape == ref.shape and got.dtype == np.dtype(dt)
            assert_close(got.get(), ref, tol, 'conv_transpose ' + what)
            routines.ROUTE_CONV_TRANSPOSE_HERE = True
            try:  # the same route issued kernel call by kernel call from the routine layer: the same kernels, the same bits
                here = chx.conv_transpose(chx.array(x), chx.array(w), bd, st, pd, out_size)
            finally:
                routines.ROUTE_CONV_TRANSPOSE_HERE = False
            assert_exact(got.get(), here.get(), 'entry against routine-level routing ' + what)
        # operands that are views: channels-last x, a w with padded strides
        wv = upload_view(chx, padded(w.shape, w, 1, dt))
        got = chx.conv_transpose(channels_last(chx, x), wv, None, st, pd, out_size)
        assert_close(got.get(), O.conv_transpose(x, w, None, st, pd, out_size), tol, 'conv_transpose of views ' + what)


def test_conv_transpose_entry_checks():
    import chainer_amd as chx
    from chainer_amd import _lib, routines
    x = chx.array(np.zeros((2, 4, 5, 5), 'float32'))
    w = chx.array(np.zeros((4, 3, 3, 3), 'float32'))
    out = chx.ndarray.empty((2, 3, 9, 9), 'float32')
    st, pd = routines._i64((2, 2)), routines._i64((1, 1))
    need = _lib.load().hipcx_conv_transpose_workspace_size(x.desc(), w.desc(), st, pd, out.desc())
    assert need > 0
    with pytest.raises(chx.ChainerxError):  # no workspace
        _lib.call('hipcx_conv_transpose', x.desc(), w.desc(), None, st, pd, out.desc(), None, 0, None)
    bad = chx.ndarray.empty((2, 3, 20, 20), 'float32')
    assert _lib.load().hipcx_conv_transpose_workspace_size(x.desc(), w.desc(), st, pd, bad.desc()) == 0
    ws = chx.alloc_bytes(need)
    with pytest.raises(chx.DimensionError):
        _lib.call('hipcx_conv_transpose', x.desc(), w.desc(), None, st, pd, bad.desc(), ws.data_ptr(), need, None)
    with pytest.raises(chx.DtypeError):
        _lib.call('hipcx_conv_transpose', x.desc(), chx.array(np.zeros((4, 3, 3, 3), 'float16')).desc(), None, st, pd, out.desc(),
                  ws.data_ptr(), need, None)


def test_batch_norm_supported_predicate():
    import ctypes
    import chainer_amd as chx
    from chainer_amd import _lib
    lib = _lib.load()

    def pointers(*arrays):
        for a in arrays:
            a.desc()  # builds the descriptor
        return (ctypes.POINTER(_lib.CArray) * len(arrays))(*[ctypes.pointer(a._desc) for a in arrays])

    x = chx.array(np.zeros((4, 6, 5, 5), 'float32'))
    g, bta = chx.array(np.ones(6, 'float32')), chx.array(np.ones((1, 6, 1, 1), 'float32'))
    axes = (ctypes.c_int8 * 3)(0, 2, 3)
    assert lib.hipcx_batch_norm_supported(x.desc(), axes, 3, pointers(g, bta), 2) == 1
    assert lib.hipcx_batch_norm_supported(x.desc(), (ctypes.c_int8 * 2)(0, 2), 2, pointers(g, bta), 2) == 0  # another axis set
    assert lib.hipcx_batch_norm_supported(x.transpose((0, 1, 3, 2)).desc(), axes, 3, pointers(g), 1) == 0      # not C-contiguous
    assert lib.hipcx_batch_norm_supported(x.desc(), axes, 3, pointers(chx.array(np.ones(6, 'float16'))), 1) == 0  # another dtype
    assert lib.hipcx_batch_norm_supported(x.desc(), axes, 3, pointers(chx.array(np.ones(5, 'float32'))), 1) == 0  # wrong length

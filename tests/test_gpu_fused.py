"""The opt-in fused entry points against the compositions of the reference's separate kernels evaluated by the CPU oracle:
hipcx_conv_bn_act (conv -> fixed_batch_norm -> add -> relu), hipcx_log_softmax (the seven-kernel LogSoftmax chain) and
hipcx_lstm_cell (the Lstm routine)."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, channels_last, padded, upload_view

pytestmark = pytest.mark.gpu


def ref_block(x, w, b, stride, pad, bn, residual, relu):
    y = O.conv(x, w, b, stride, pad)
    if bn is not None:
        y = O.fixed_batch_norm(y, *bn, 2e-5, (0, 2, 3))
    if residual is not None:
        y = O.add(y, residual)
    return O.relu(y) if relu else y


CASES = [  # N, C, H, W, K, R, stride, pad
    (2, 64, 8, 8, 64, 1, 1, 0), (3, 32, 14, 14, 128, 1, 2, 0), (2, 16, 12, 12, 32, 3, 1, 1), (4, 64, 7, 7, 256, 1, 1, 0),
    (2, 128, 7, 7, 128, 3, 1, 1), (1, 3, 20, 20, 16, 7, 2, 3), (2, 24, 6, 6, 40, 3, 2, 1), (2, 3, 32, 32, 64, 7, 2, 3),
]


@pytest.mark.parametrize('dt,tol', [('float16', 2e-2), ('float32', 1e-5)])
def test_conv_bn_act_matches_composition(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(0)
    for (N, C, H, W, K, R, st, pd) in CASES:
        x = rng.standard_normal((N, C, H, W)).astype(dt)
        w = (rng.standard_normal((K, C, R, R)) / np.sqrt(C * R * R)).astype(dt)
        b = rng.standard_normal(K).astype(dt)
        bn = [rng.uniform(0.5, 1.5, K).astype(dt), (rng.standard_normal(K) * 0.1).astype(dt), (rng.standard_normal(K) * 0.1).astype(dt),
              rng.uniform(0.5, 1.5, K).astype(dt)]
        oh = (H + 2 * pd - R) // st + 1
        res = rng.standard_normal((N, K, oh, oh)).astype(dt)
        for use_bn, use_res, relu, bias in [(True, True, True, False), (True, False, True, False), (True, False, False, True),
                                            (False, True, True, True), (False, False, False, False)]:
            ref = ref_block(x, w, b if bias else None, st, pd, bn if use_bn else None, res if use_res else None, relu)
            for lay, X in (('nchw', chx.array(x)), ('nhwc', channels_last(chx, x))):
                y = chx.conv_bn_act(X, chx.array(w), chx.array(b) if bias else None, st, pd, False,
                                    [chx.array(a) for a in bn] if use_bn else None, 2e-5, chx.array(res) if use_res else None, relu)
                assert_close(y.get(), ref, tol, '%s %s bn=%s res=%s relu=%s %s' % (dt, lay, use_bn, use_res, relu, (N, C, H, W, K, R, st, pd)))


def test_relu_lets_nan_through_and_params_may_be_keepdims():
    import chainer_amd as chx
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 32, 4, 4)).astype('float16')
    x[0, 0, 1, 1] = np.nan
    w = (rng.standard_normal((32, 32, 1, 1)) / 6).astype('float16')
    bn = [np.ones(32, 'float16'), np.zeros(32, 'float16'), np.zeros(32, 'float16'), np.ones(32, 'float16')]
    y = chx.conv_bn_act(chx.array(x), chx.array(w), None, 1, 0, False, [chx.array(a.reshape(1, 32, 1, 1)) for a in bn], 2e-5, None, True).get()
    ref = ref_block(x, w, None, 1, 0, bn, None, True)
    assert np.isnan(y[0, :, 1, 1]).all() and np.array_equal(np.isnan(y), np.isnan(ref))
    with pytest.raises(chx.DimensionError):
        chx.conv_bn_act(chx.array(x), chx.array(w), None, 1, 0, False, [chx.array(a[:5]) for a in bn], 2e-5, None, True)


def test_resnet50_fused_forward():
    """The fused network against the oracle's unfused one (batch 2), and against the unfused hip path at batch 16."""
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p = cfg.resnet50_params()
    pd = cfg.tree_map(chx.array, p)
    x = cfg.resnet50_input(batch=16)
    ref = cfg.resnet50_forward(O, p, x[:2])
    y = cfg.resnet50_forward_fused(chx, pd, chx.array(x[:2])).get()
    assert_close(y, ref, 2e-2, 'fused vs oracle')
    assert np.array_equal(y.argmax(1), ref.argmax(1))
    y16 = cfg.resnet50_forward_fused(chx, pd, chx.array(x)).get()
    u16 = cfg.resnet50_forward(chx, pd, chx.array(x)).get()
    assert_close(y16, u16, 2e-2, 'fused vs unfused hip')


LSM_SHAPES = [  # float32 rows up to 16384 elements stay in registers; longer ones take the two-pass kernels
    (100, 10), (7, 1), (1, 3), (64, 4096), (5, 10000), (3, 16384), (2, 16385), (3, 200000), (9, 257), (4, 1025),
]


@pytest.mark.parametrize('dt', ['float32', 'float16', 'float64'])
def test_log_softmax_fused_matches_chain(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(11)
    for shape in LSM_SHAPES:
        x = (rng.standard_normal(shape) * 3).astype(dt)
        ref = O.log_softmax(x, 1)
        got = chx.log_softmax_fused(chx.array(x), 1).get()
        assert_close(got, ref, None, 'log_softmax_fused %s %s' % (dt, shape))
        # rows of exp(out) sum to one (float16 outputs carry half an ulp of -log(n) each)
        total = np.exp(got.astype(np.float64)).sum(axis=1)
        assert np.allclose(total, 1.0, rtol=0, atol={'float16': 2e-2, 'float32': 1e-5, 'float64': 1e-12}[dt]), (dt, shape)
    # against the seven separate kernels on the device
    x = (rng.standard_normal((33, 1000)) * 2).astype(dt)
    assert_close(chx.log_softmax_fused(chx.array(x)).get(), chx.log_softmax(chx.array(x)).get(), None, 'fused vs chain on the device')


def test_log_softmax_fused_views_and_special_values():
    import chainer_amd as chx
    rng = np.random.default_rng(12)
    # rows with a pitch (non-contiguous, unaligned): a padded parent array
    for shape in [(6, 37), (5, 70001)]:
        x = padded(shape, rng.standard_normal(shape), 1, 'float32')
        assert not x.flags.c_contiguous
        assert_close(chx.log_softmax_fused(upload_view(chx, x)).get(), O.log_softmax(x, 1), None, 'padded rows %r' % (shape,))
    # NaN poisons its row, -inf entries drop out, a row of -inf only and a row holding +inf become NaN (as in the chain)
    for n in (50, 40000):
        x = rng.standard_normal((6, n)).astype('float32')
        x[1, n // 2] = np.nan
        x[2, : n // 3] = -np.inf
        x[3, :] = -np.inf
        x[4, 7] = np.inf
        if n > 20000:
            x[5, :16384] = -np.inf  # a whole -inf segment of the two-pass kernel inside a finite row
        ref = O.log_softmax(x, 1)
        got = chx.log_softmax_fused(chx.array(x)).get()
        assert_close(got, ref, None, 'special values n=%d' % n)
        assert np.isnan(got[1]).all() and np.isnan(got[3]).all() and np.isnan(got[4]).all()
        assert np.isfinite(got[0]).all() and np.isfinite(got[5, -1])
    # other axes / ranks fall back to the chain
    x3 = rng.standard_normal((3, 4, 5)).astype('float32')
    assert_close(chx.log_softmax_fused(chx.array(x3), 2).get(), O.log_softmax(x3, 2), None, '3-D')
    x2 = rng.standard_normal((8, 9)).astype('float32')
    assert_close(chx.log_softmax_fused(chx.array(x2), 0).get(), O.log_softmax(x2, 0), None, 'axis 0')
    assert chx.log_softmax_fused(chx.array(np.zeros((0, 5), 'float32'))).shape == (0, 5)
    with pytest.raises(chx.DtypeError):
        chx._lib.call('hipcx_log_softmax', chx.array(np.zeros((2, 2), 'int32')).desc(), chx.array(np.zeros((2, 2), 'int32')).desc(), None, 0,
                      chx.routines.current_stream())


@pytest.mark.parametrize('dt', ['float32', 'float64', 'float16'])
def test_lstm_cell_fused(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(13)
    for (B, H) in [(128, 650), (1, 1), (3, 7), (64, 33), (5, 1024)]:
        c = rng.standard_normal((B, H)).astype(dt)
        x = (rng.standard_normal((B, 4 * H)) * 2).astype(dt)
        h_ref, c_ref = O.lstm(c, x)
        h, cn = chx.lstm_fused(chx.array(c), chx.array(x))
        assert_close(h.get(), h_ref, None, 'lstm h %s %r' % (dt, (B, H)))
        assert_close(cn.get(), c_ref, None, 'lstm c %s %r' % (dt, (B, H)))
        if dt != 'float16':  # same operations in the same order as the ~25 separate kernels
            h2, c2 = chx.lstm(chx.array(c), chx.array(x))
            assert_exact(h.get(), h2.get(), 'fused h vs chain')
            assert_exact(cn.get(), c2.get(), 'fused c vs chain')
    # strided rows: c and x as column blocks of wider arrays
    big = rng.standard_normal((6, 50)).astype(dt)
    c_v, x_v = big[:, 3:10], big[:, 12:40]
    h, cn = chx.lstm_fused(upload_view(chx, c_v), upload_view(chx, x_v))
    h_ref, c_ref = O.lstm(c_v, x_v)
    assert_close(h.get(), h_ref, None, 'lstm strided h')
    assert_close(cn.get(), c_ref, None, 'lstm strided c')


def test_lstm_cell_fused_errors():
    """Shape and dtype errors of the Lstm routine (CX/routines/connection.cc:398-416)."""
    import chainer_amd as chx
    z = lambda shape, dt='float32': chx.array(np.zeros(shape, dt))
    with pytest.raises(chx.DimensionError):
        chx.lstm_fused(z((2, 3)), z((2, 11)))
    with pytest.raises(chx.DimensionError):
        chx.lstm_fused(z((2, 3)), z((3, 12)))
    with pytest.raises(chx.DtypeError):
        chx.lstm_fused(z((2, 3), 'int32'), z((2, 12), 'int32'))
    with pytest.raises(chx.DtypeError):
        chx.lstm_fused(z((2, 3), 'float32'), z((2, 12), 'float64'))

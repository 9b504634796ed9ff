"""The backward / training kernels (ConvGradWeight, ConvTranspose, BatchNorm + BatchNormGrad, MaxPoolGrad, AveragePoolGrad),
composed on the device from the forward kernels the way the reference's native backend composes them, against the CPU oracle.

Bar: 1e-5 relative float32, 2e-2 float16, 1e-12 float64 for everything that goes through Dot; the pooling gradients add in
the reference's order and are held to the same tolerances."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact, channels_last

pytestmark = pytest.mark.gpu

DT = [('float32', 1e-5), ('float16', 2e-2), ('float64', 1e-12)]
CONV_CASES = [  # N, C, H, W, K, kh, kw, stride, pad, cover_all
    (2, 3, 9, 8, 4, 3, 3, (2, 1), (1, 2), False), (2, 16, 8, 8, 32, 3, 3, 1, 1, False), (3, 64, 7, 7, 64, 1, 1, 1, 0, False),
    (2, 32, 10, 10, 24, 3, 3, 2, 1, True), (1, 3, 20, 20, 8, 7, 7, 2, 3, False), (2, 20, 6, 7, 9, 2, 3, (1, 2), (0, 1), False),
    (4, 8, 12, 12, 16, 1, 1, 2, 0, False),
    # 1x1 filters at a stride: ConvTranspose runs as a 1x1 convolution scattered into a zero-filled output
    (2, 16, 13, 9, 8, 1, 1, (2, 3), 0, False), (2, 8, 10, 10, 8, 1, 1, 2, 0, True), (2, 256, 14, 14, 512, 1, 1, 2, 0, False),
    # 1x1 filters at stride 1 on planes of whole 16-byte granules: ConvGradWeight reads gy and x in place, one matrix product per
    # image accumulated (one slice; a split reduction; a last reduction step that is partly past the plane; float32-only granules)
    (3, 32, 16, 16, 48, 1, 1, 1, 0, False), (16, 64, 28, 28, 256, 1, 1, 1, 0, False), (2, 200, 28, 28, 72, 1, 1, 1, 0, False),
    (2, 24, 18, 18, 40, 1, 1, 1, 0, False),
    # stride 1: ConvTranspose runs as a forward convolution with flipped filters (padding k - 1 - p)
    (2, 6, 7, 9, 10, 2, 3, 1, (0, 1), False), (2, 8, 9, 9, 12, 5, 5, 1, 2, False), (2, 16, 6, 6, 16, 3, 3, 1, 0, False),
    (4, 64, 14, 14, 128, 3, 3, 1, 1, False), (2, 128, 7, 7, 256, 1, 1, 1, 0, False), (2, 5, 6, 6, 7, 3, 3, 1, 2, False),
    # filters larger than 1x1 at stride 1 in float16 / float32: ConvGradWeight multiplies gy with windows of shifted zero-padded
    # copies of x (planes wider than the padded row granule, non-square planes and filters, one-sided padding, a reduction
    # split over many slices, channel counts that are no multiple of a tile)
    (2, 64, 28, 28, 64, 3, 3, 1, 1, False), (3, 16, 12, 20, 24, 3, 3, 1, 1, False), (2, 8, 10, 12, 8, 3, 5, 1, (1, 2), False),
    (16, 64, 14, 14, 64, 3, 3, 1, 1, False), (2, 13, 15, 17, 21, 3, 3, 1, (1, 0), False), (1, 8, 30, 30, 8, 2, 2, 1, 0, False),
]


@pytest.mark.parametrize('dt,tol', DT)
def test_conv_grad_weight_and_transpose(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(50)
    for (N, C, H, W, K, kh, kw, st, pd, cv) in CONV_CASES:
        x = rng.standard_normal((N, C, H, W)).astype(dt)
        w = (rng.standard_normal((K, C, kh, kw)) / np.sqrt(C * kh * kw)).astype(dt)
        y_shape = O.conv(x.astype('float32'), w.astype('float32'), None, st, pd, cv).shape
        gy = (rng.standard_normal(y_shape) / np.sqrt(K)).astype(dt)
        what = '%s %r' % (dt, (N, C, H, W, K, kh, kw, st, pd, cv))
        gw = chx.conv_grad_weight(dt, w.shape, chx.array(x), chx.array(gy), st, pd, cv)
        assert gw.shape == w.shape and gw.dtype == np.dtype(dt)
        assert_close(gw.get(), O.conv_grad_weight(w.shape, x, gy, st, pd, cv), tol, 'conv_grad_weight ' + what)
        from chainer_amd import routines
        routines.COMPOSE_CONV_GRAD_WEIGHT = True
        try:  # the same product issued as strided copies + Dot from the routine layer
            gw_c = chx.conv_grad_weight(dt, w.shape, chx.array(x), chx.array(gy), st, pd, cv)
        finally:
            routines.COMPOSE_CONV_GRAD_WEIGHT = False
        assert_close(gw_c.get(), O.conv_grad_weight(w.shape, x, gy, st, pd, cv), tol, 'conv_grad_weight (composed) ' + what)
        gw_v = chx.conv_grad_weight(dt, w.shape, channels_last(chx, x), chx.array(gy), st, pd, cv)  # a non-contiguous x is copied first
        assert_close(gw_v.get(), O.conv_grad_weight(w.shape, x, gy, st, pd, cv), tol, 'conv_grad_weight (channels-last x) ' + what)
        gx = chx.conv_transpose(chx.array(gy), chx.array(w), None, st, pd, (H, W))
        assert gx.shape == x.shape
        assert_close(gx.get(), O.conv_transpose(gy, w, None, st, pd, (H, W)), tol, 'conv_transpose ' + what)
        b = rng.standard_normal(C).astype(dt)
        assert_close(chx.conv_transpose(chx.array(gy), chx.array(w), chx.array(b), st, pd, (H, W)).get(),
                     O.conv_transpose(gy, w, b, st, pd, (H, W)), tol, 'conv_transpose + bias ' + what)
    # default output size and the shape checks of the routine
    gy = rng.standard_normal((2, 4, 5, 5)).astype(dt)
    w = rng.standard_normal((4, 3, 3, 3)).astype(dt)
    out = chx.conv_transpose(chx.array(gy), chx.array(w), None, 2, 1)
    assert out.shape == (2, 3, 9, 9)
    assert_close(out.get(), O.conv_transpose(gy, w, None, 2, 1), tol, 'default out_size')
    with pytest.raises(chx.DimensionError):
        chx.conv_transpose(chx.array(gy), chx.array(w[:3]), None, 2, 1)
    with pytest.raises(chx.DimensionError):
        chx.conv_transpose(chx.array(gy), chx.array(w), None, 2, 1, (20, 20))


def test_conv_backward_is_the_adjoint_on_the_device():
    """<conv(x, w), gy> = <x, conv_transpose(gy, w)> = <w, conv_grad_weight(x, gy)> with all three evaluated on the device."""
    import chainer_amd as chx
    rng = np.random.default_rng(51)
    x = rng.standard_normal((4, 16, 14, 14)).astype('float32')
    w = (rng.standard_normal((32, 16, 3, 3)) / 12).astype('float32')
    X, Wd = chx.array(x), chx.array(w)
    y = chx.conv(X, Wd, None, 1, 1)
    gy = rng.standard_normal(y.shape).astype('float32')
    G = chx.array(gy)
    lhs = float((y.get().astype(np.float64) * gy).sum())
    gx = chx.conv_transpose(G, Wd, None, 1, 1, (14, 14)).get().astype(np.float64)
    gw = chx.conv_grad_weight('float32', w.shape, X, G, 1, 1).get().astype(np.float64)
    assert abs((x * gx).sum() - lhs) <= 1e-4 * abs(lhs) + 1e-3
    assert abs((w * gw).sum() - lhs) <= 1e-4 * abs(lhs) + 1e-3


@pytest.mark.parametrize('dt,tol', DT)
def test_batch_norm_training_and_grad(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(52)
    for shape in [(8, 6, 5, 4), (16, 3, 7, 7), (32, 10)]:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + 0.5).astype(dt)
        gamma, beta = rng.uniform(0.5, 1.5, C).astype(dt), (rng.standard_normal(C) * 0.1).astype(dt)
        rm, rv = (rng.standard_normal(C) * 0.1).astype(dt), rng.uniform(0.5, 1.5, C).astype(dt)
        axis = (0,) if len(shape) == 2 else None
        RM, RV = chx.array(rm), chx.array(rv)
        out, state = chx.batch_norm(chx.array(x), chx.array(gamma), chx.array(beta), RM, RV, 2e-5, 0.9, axis)
        o_ref, rm_ref, rv_ref, st_ref = O.batch_norm(x, gamma, beta, rm, rv, 2e-5, 0.9, axis)
        assert_close(out.get(), o_ref, tol, 'batch_norm out %s %r' % (dt, shape))
        assert_close(RM.get(), rm_ref, tol, 'running mean (updated in place)')
        assert_close(RV.get(), rv_ref, tol, 'running var (updated in place)')
        gout = rng.standard_normal(shape).astype(dt)
        gx, gg, gb = chx.batch_norm_grad(chx.array(x), chx.array(gamma), chx.array(gout), state, axis)
        gx_ref, gg_ref, gb_ref = O.batch_norm_grad(x, gamma, gout, st_ref, axis)
        gtol = tol * (50 if dt == 'float16' else 20)  # the gradient cancels terms of size |gout| * n
        assert_close(gx.get(), gx_ref, gtol, 'batch_norm gx')
        assert_close(gg.get(), gg_ref, gtol, 'batch_norm ggamma')
        assert_close(gb.get(), gb_ref, gtol, 'batch_norm gbeta')
    with pytest.raises(chx.DtypeError):
        chx.batch_norm(chx.array(np.zeros((2, 3), 'int32')), chx.array(np.ones(3, 'float32')), chx.array(np.ones(3, 'float32')),
                       chx.array(np.ones(3, 'float32')), chx.array(np.ones(3, 'float32')), axis=(0,))


POOL_CASES = [((2, 3, 7, 6), (3, 3), (2, 2), (1, 1), False), ((1, 2, 5, 5), (2, 3), (1, 2), (0, 1), True), ((2, 4, 8, 8), (2, 2), (2, 2), (0, 0), False),
              ((2, 8, 14, 14), (3, 3), (2, 2), (1, 1), False), ((3, 5, 9, 9), (3, 3), (1, 1), (1, 1), False)]


@pytest.mark.parametrize('dt,tol', DT)
def test_pool_grads(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(53)
    for (shape, k, s, p, cv) in POOL_CASES:
        x = rng.integers(-4, 5, shape).astype(dt)  # ties inside windows: the ArgMax tie rule decides
        y_shape = O.max_pool(x, k, s, p, cv).shape
        g = rng.standard_normal(y_shape).astype(dt)
        gx = chx.max_pool_grad(chx.array(x), chx.array(g), k, s, p, cv)
        assert gx.shape == x.shape
        if dt == 'float16':
            assert_close(gx.get(), O.max_pool_grad(x, g, k, s, p, cv), tol, 'max_pool_grad %r' % (shape,))
        else:  # same additions in the same order
            assert_exact(gx.get(), O.max_pool_grad(x, g, k, s, p, cv), 'max_pool_grad %r' % (shape,))
        if not cv:
            xf = rng.standard_normal(shape).astype(dt)
            for mode in ('zero', 'ignore'):
                ya = O.average_pool(xf, k, s, p, mode)
                ga = rng.standard_normal(ya.shape).astype(dt)
                got = chx.average_pool_grad(chx.array(xf), chx.array(ga), k, s, p, mode)
                assert_close(got.get(), O.average_pool_grad(xf, ga, k, s, p, mode), tol, 'average_pool_grad %s %r' % (mode, shape))


def test_var_routine():
    import chainer_amd as chx
    rng = np.random.default_rng(54)
    x = rng.standard_normal((6, 5, 40)).astype('float32')
    assert_close(chx.var(chx.array(x), (0, 2)).get(), O.var(x, (0, 2)), 1e-5, 'var')
    assert_close(chx.var(chx.array(x), 1, True).get(), O.var(x, 1, True), 1e-5, 'var keepdims')


def test_max_pool_grad_grad_and_nanarg():
    import chainer_amd as chx
    rng = np.random.default_rng(55)
    for (shape, k, s, p, cv) in POOL_CASES:
        x = rng.integers(-4, 5, shape).astype('float32')
        ggx = rng.standard_normal(shape).astype('float32')
        got = chx.max_pool_grad_grad(chx.array(x), chx.array(ggx), k, s, p, cv)
        assert_exact(got.get(), O.max_pool_grad_grad(x, ggx, k, s, p, cv), 'max_pool_grad_grad %r' % (shape,))
    # for tie-free x the double gradient of the gradient's own input is the pooled value itself
    xt = rng.standard_normal((2, 3, 8, 8)).astype('float32')
    assert_exact(chx.max_pool_grad_grad(chx.array(xt), chx.array(xt), 2, 2, 0).get(), O.max_pool(xt, 2, 2, 0), 'ggx = x gives max_pool(x)')
    a = rng.standard_normal((5, 200)).astype('float32')
    a[0, 3] = np.nan
    a[1, :] = np.nan
    a[2, 0] = np.nan
    assert_exact(chx.nanargmax(chx.array(a), 1).get(), O.nanargmax(a, 1), 'nanargmax')
    assert_exact(chx.nanargmin(chx.array(a), 1).get(), O.nanargmin(a, 1), 'nanargmin')
    assert chx.nanargmax(chx.array(a), 1).get()[0] == np.nanargmax(a[0]) and chx.nanargmin(chx.array(a), 1).get()[2] == np.nanargmin(a[2])


@pytest.mark.parametrize('dt', ['float32', 'float16', 'float64', 'int32'])
def test_pool_gradient_kernels_have_the_bits_of_the_composition(dt):
    """hipcx_max_pool_grad / hipcx_average_pool_grad against the Im2Col / ArgMax / Col2Im composition on the device: same
    additions in the same order, same ArgMax choice among ties and NaNs (a 7x7 window crosses the 32-element block of the
    reduction tree), for dense, channels-last and overlapping / non-overlapping windows."""
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(61)
    cases = POOL_CASES + [((2, 3, 20, 20), 7, 3, 3, False), ((1, 2, 15, 15), 7, 1, 0, False), ((2, 4, 9, 11), (3, 2), (1, 2), (1, 0), True),
                          ((3, 5, 12, 12), 3, 2, 1, False), ((2, 8, 56, 56), 3, 2, 1, False),
                          # stride-2 windows over planes whose width is a multiple of 8 with OW = W / 2 (vector kernels): 3x3 without
                          # padding (cover_all), 2x2, a vertical stride of 3, several octets per row
                          ((2, 3, 16, 16), 3, 2, 0, True), ((2, 3, 16, 24), 2, 2, 0, False), ((1, 2, 12, 16), 3, (3, 2), (1, 1), False),
                          ((2, 2, 14, 40), 3, 2, 1, False),
                          # windows that are the whole plane (the global pooling of a classifier head): planes of 49, 30 and 9 elements
                          ((3, 5, 7, 7), 7, 1, 0, False), ((2, 3, 6, 5), (6, 5), 1, 0, False), ((1, 1, 3, 3), 3, 3, 0, False)]
    for (shape, k, s, p, cv) in cases:
        x = rng.integers(-3, 4, shape).astype(dt)
        if np.dtype(dt).kind == 'f':
            x[rng.random(shape) < 0.05] = np.nan
        y_shape = O.max_pool(np.nan_to_num(x), k, s, p, cv).shape
        g = rng.standard_normal(y_shape).astype(dt) if np.dtype(dt).kind == 'f' else rng.integers(-50, 50, y_shape).astype(dt)
        for lay in ('nchw', 'nhwc'):
            X = chx.array(x) if lay == 'nchw' else channels_last(chx, x)
            G = chx.array(g) if lay == 'nchw' else channels_last(chx, g)
            got = chx.max_pool_grad(X, G, k, s, p, cv).get()
            routines.COMPOSE_POOL_GRADIENTS = True
            try:
                ref = chx.max_pool_grad(X, G, k, s, p, cv).get()
            finally:
                routines.COMPOSE_POOL_GRADIENTS = False
            assert_exact(got, ref, 'max_pool_grad %s %s %r' % (dt, lay, (shape, k, s, p, cv)))
            ggx = rng.standard_normal(shape).astype(dt) if np.dtype(dt).kind == 'f' else rng.integers(-50, 50, shape).astype(dt)
            GGX = chx.array(ggx) if lay == 'nchw' else channels_last(chx, ggx)
            got = chx.max_pool_grad_grad(X, GGX, k, s, p, cv).get()
            routines.COMPOSE_POOL_GRADIENTS = True
            try:
                ref = chx.max_pool_grad_grad(X, GGX, k, s, p, cv).get()
            finally:
                routines.COMPOSE_POOL_GRADIENTS = False
            assert_exact(got, ref, 'max_pool_grad_grad %s %s %r' % (dt, lay, (shape, k, s, p, cv)))
        if np.dtype(dt).kind == 'f' and not cv:
            for mode in ('zero', 'ignore'):
                got = chx.average_pool_grad(chx.array(x), chx.array(g), k, s, p, mode).get()
                routines.COMPOSE_POOL_GRADIENTS = True
                try:
                    ref = chx.average_pool_grad(chx.array(x), chx.array(g), k, s, p, mode).get()
                finally:
                    routines.COMPOSE_POOL_GRADIENTS = False
                assert_exact(got, ref, 'average_pool_grad %s %s %r' % (dt, mode, (shape, k, s, p)))
    with pytest.raises(chx.DimensionError):
        chx.max_pool_grad(chx.zeros((1, 1, 4, 4), dt), chx.zeros((1, 1, 3, 3), dt), 2, 2, 0)


@pytest.mark.parametrize('dt,tol', [('float32', 1e-5), ('float16', 2e-2), ('float64', 1e-12)])
def test_batch_norm_kernels_against_the_composition(dt, tol):
    """hipcx_batch_norm / hipcx_batch_norm_grad against the reference's routine composition on the device and against the oracle:
    plane sizes that are and are not whole 16-byte vectors, one image, one channel, 2-D input, a large-mean input (the two-pass
    variance must not cancel), running statistics updated in place; a non-contiguous x takes the composition."""
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(71)
    shapes = [(8, 16, 14, 14), (4, 3, 7, 7), (1, 5, 6, 4), (6, 1, 3, 3), (32, 10), (2, 4, 3, 5, 2), (16, 8, 7, 7), (3, 24, 14, 14),
              (5, 7, 3, 3)]
    if dt != 'float16':
        # 50176 elements per channel: the float16 composition (like the native backend) overflows its Sum of squares there and
        # returns inf statistics; test_batch_norm_float16_overflow covers that case
        shapes.append((64, 32, 28, 28))
    for shape in shapes:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + (5 if shape == (4, 3, 7, 7) else 0)).astype(dt)
        gamma = rng.uniform(0.5, 1.5, C).astype(dt)
        beta = rng.standard_normal(C).astype(dt)
        rm0, rv0 = rng.standard_normal(C).astype(dt), rng.uniform(0.5, 1.5, C).astype(dt)
        gout = rng.standard_normal(shape).astype(dt)
        res = {}
        for mode in ('kernel', 'composition'):
            routines.COMPOSE_BATCH_NORM = mode == 'composition'
            try:
                RM, RV = chx.array(rm0), chx.array(rv0)
                out, state = chx.batch_norm(chx.array(x), chx.array(gamma), chx.array(beta), RM, RV, 2e-5, 0.9)
                gx, gg, gb = chx.batch_norm_grad(chx.array(x), chx.array(gamma), chx.array(gout), state)
                res[mode] = [out.get(), RM.get(), RV.get(), state[0].get(), state[1].get(), gx.get(), gg.get(), gb.get()]
            finally:
                routines.COMPOSE_BATCH_NORM = False
        names = ['out', 'running_mean', 'running_var', 'mean', 'inv_std']
        for name, a, b in zip(names, res['kernel'], res['composition']):
            assert_close(a, b, tol, 'batch_norm %s %s %r kernel vs composition' % (name, dt, shape))
        # gradients against the closed form in float64; the sums cancel, so errors are measured against the size of their terms
        red = (0,) + tuple(range(2, x.ndim))
        bshape = (1, C) + (1,) * (x.ndim - 2)
        x64, g64 = x.astype(np.float64), gout.astype(np.float64)
        m64 = x64.mean(red, keepdims=True)
        is64 = 1.0 / np.sqrt(x64.var(red, keepdims=True) + 2e-5)
        xh = (x64 - m64) * is64
        gb64, gg64 = g64.sum(red), (g64 * xh).sum(red)
        gx64 = gamma.astype(np.float64).reshape(bshape) * is64 * (g64 - (xh * gg64.reshape(bshape) + gb64.reshape(bshape)) / (x.size // C))
        gx, gg, gb = res['kernel'][5:8]
        t = 4 * tol
        assert gx.dtype == x.dtype and gg.shape == (C,) and gb.shape == (C,)
        assert np.all(np.abs(gb.astype(np.float64) - gb64) <= t * np.abs(g64).sum(red) + 1e-30), 'gbeta %s %r' % (dt, shape)
        assert np.all(np.abs(gg.astype(np.float64) - gg64) <= t * np.abs(g64 * xh).sum(red) + 1e-30), 'ggamma %s %r' % (dt, shape)
        assert np.abs(gx.astype(np.float64) - gx64).max() <= t * np.abs(gx64).max() + t * 1e-2, 'gx %s %r' % (dt, shape)
        o_ref, rm_ref, rv_ref, st_ref = O.batch_norm(x, gamma, beta, rm0.copy(), rv0.copy(), 2e-5, 0.9)
        assert_close(res['kernel'][0], o_ref, tol, 'batch_norm out vs oracle %s %r' % (dt, shape))
        assert_close(res['kernel'][1], rm_ref, tol, 'running_mean vs oracle')
        assert_close(res['kernel'][2], rv_ref, tol, 'running_var vs oracle')
    # a channels-last view is not C-contiguous: the composition runs and agrees
    x = rng.standard_normal((4, 8, 5, 5)).astype(dt)
    X = channels_last(chx, x)
    g1, b1 = np.ones(8, dt), np.zeros(8, dt)
    out, _ = chx.batch_norm(X, chx.array(g1), chx.array(b1), chx.array(b1.copy()), chx.array(g1.copy()))
    assert_close(out.get(), O.batch_norm(x, g1, b1, b1.copy(), g1.copy(), 2e-5, 0.9)[0], tol, 'channels-last input')


@pytest.mark.parametrize('case', ['sum of squares', 'sum', 'square', 'finite'])
def test_batch_norm_float16_overflow(case):
    """The reference's float16 BatchNorm is a composition of float16 routines (CX/routines/normalization.cc:155-193): its Sum hands
    out a float16 (inf past 65504), (x - mean)^2 is a float16 array, and everything after an inf follows IEEE rules.  The kernels
    give the same special values in the same places as the oracle and as the composition run on the device: a variance of inf
    (inv_std 0, out == beta), a mean of inf (out NaN), one squared deviation of inf in an otherwise small channel, and -- as the
    control -- the same shape with finite statistics."""
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(171)
    shape = (64, 6, 28, 28)  # 50176 elements per channel
    x = rng.standard_normal(shape)
    if case == 'sum of squares':
        x = x * 2                      # sum (x - mean)^2 is about 2e5
    elif case == 'sum':
        x = x * 0.25 + 3               # sum x is about 1.5e5
    elif case == 'square':
        x = x * 0.05
        x[3, 2, 5, 7] = 300.0          # (x - mean)^2 = 9e4 rounds to inf in channel 2 only
    else:
        x = x * 0.05 + 0.01
    x = x.astype(np.float16)
    C = shape[1]
    gamma, beta = rng.uniform(0.5, 1.5, C).astype(np.float16), rng.standard_normal(C).astype(np.float16)
    rm0, rv0 = rng.standard_normal(C).astype(np.float16), rng.uniform(0.5, 1.5, C).astype(np.float16)
    gout = (rng.standard_normal(shape) * 0.1).astype(np.float16)
    res = {}
    for mode in ('kernel', 'composition'):
        routines.COMPOSE_BATCH_NORM = mode == 'composition'
        try:
            RM, RV = chx.array(rm0), chx.array(rv0)
            out, state = chx.batch_norm(chx.array(x), chx.array(gamma), chx.array(beta), RM, RV, 2e-5, 0.9)
            gx, gg, gb = chx.batch_norm_grad(chx.array(x), chx.array(gamma), chx.array(gout), state)
            res[mode] = [out.get(), RM.get(), RV.get(), state[0].get(), state[1].get(), gx.get(), gg.get(), gb.get()]
        finally:
            routines.COMPOSE_BATCH_NORM = False
    o_ref, rm_ref, rv_ref, st_ref = O.batch_norm(x, gamma, beta, rm0.copy(), rv0.copy(), 2e-5, 0.9)
    gx_ref, gg_ref, gb_ref = O.batch_norm_grad(x, gamma, gout, st_ref)
    ref = [o_ref, rm_ref, rv_ref, st_ref[0].reshape(C), st_ref[1].reshape(C), gx_ref, gg_ref.reshape(C), gb_ref.reshape(C)]
    names = ['out', 'running_mean', 'running_var', 'mean', 'inv_std', 'gx', 'ggamma', 'gbeta']
    # the case is what its name says
    if case == 'sum of squares':
        assert np.all(ref[4] == 0) and np.all(np.isinf(rv_ref)) and np.all(np.isfinite(o_ref))
    elif case == 'sum':
        assert np.all(np.isinf(ref[3])) and np.all(np.isnan(o_ref))
    elif case == 'square':
        assert ref[4][2] == 0 and np.all(ref[4][[0, 1, 3, 4, 5]] > 0)
    else:
        assert all(np.all(np.isfinite(r)) for r in ref)
    for name, k, c, r in zip(names, res['kernel'], res['composition'], ref):
        k, c = k.reshape(r.shape), c.reshape(r.shape)
        # assert_close demands the same NaN pattern and the same infinities before it compares the finite values
        tol = 5e-2 if name in ('gx', 'ggamma', 'gbeta') else 2e-2
        assert_close(k, r, tol, 'float16 batch_norm (%s) %s: kernel vs oracle' % (case, name))
        assert_close(k, c, tol, 'float16 batch_norm (%s) %s: kernel vs composition on the device' % (case, name))


@pytest.mark.parametrize('dt,tol', [('float16', 2e-2), ('float32', 1e-4)])
def test_conv_grad_weight_special_values(dt, tol):
    """inf / NaN in x on the route that reads shifted zero-padded copies of x (filters larger than 1x1 at stride 1): the filter
    taps that the reference's TensorDot(gy, Im2Col(x)) leaves finite stay finite, the others carry the same inf / NaN
    (CX/native/native_device/conv.cc:91-124).  Values planted in a corner, on an edge column (where a shifted window wraps around
    a row end) and in the interior, one channel each; an inf in gy meets the padding's zeros in both implementations."""
    import chainer_amd as chx
    rng = np.random.default_rng(190)
    for (N, C, H, W, K, kh, kw, pd) in [(4, 12, 14, 14, 16, 3, 3, 1), (2, 6, 9, 13, 8, 3, 5, (1, 2)), (3, 8, 12, 12, 8, 2, 2, 0)]:
        x = rng.standard_normal((N, C, H, W)).astype(dt)
        gy_shape = O.conv(x.astype('float32'), np.zeros((K, C, kh, kw), 'float32'), None, 1, pd).shape
        gy = np.abs(rng.standard_normal(gy_shape)).astype(dt) + np.asarray(0.25, dt)  # no zeros, one sign: inf * gy sums to inf, not NaN
        x[0, 1, 0, 0] = np.inf
        x[1, 3, 4, W - 1] = -np.inf
        x[N - 1, 4, H - 1, 0] = np.inf
        x[1, 5, H // 2, W // 2] = np.nan
        ref = O.conv_grad_weight((K, C, kh, kw), x, gy, 1, pd)
        what = '%s %r' % (dt, (N, C, H, W, K, kh, kw, pd))
        assert np.isfinite(ref[:, [0, 2]]).all() and not np.isfinite(ref[:, 1]).all(), what
        if kh == 3 and pd != 0:
            # the corner value is outside some taps' windows: those taps are finite in the reference
            assert np.isfinite(ref[:, 1]).any() and np.isinf(ref[:, 1]).any(), what
        got = chx.conv_grad_weight(dt, (K, C, kh, kw), chx.array(x), chx.array(gy), 1, pd).get()
        assert_close(got, ref, tol, 'conv_grad_weight with inf / NaN in x ' + what)  # same NaN pattern, same infinities, finite values close
        gy2 = gy.copy()
        gy2[0, 2, 0, 1] = np.inf
        x2 = rng.standard_normal((N, C, H, W)).astype(dt)
        assert_close(chx.conv_grad_weight(dt, (K, C, kh, kw), chx.array(x2), chx.array(gy2), 1, pd).get(),
                     O.conv_grad_weight((K, C, kh, kw), x2, gy2, 1, pd), tol, 'conv_grad_weight with inf in gy ' + what)


def test_batch_norm_float16_with_float32_parameters():
    """The mixed-precision call (float16 x and gout; float32 gamma, beta, running statistics): the reference computes in float32
    (CX/routines/normalization.cc:176-180) and so do the kernels -- no float16 overflow at 50176 elements per channel, state and
    parameter gradients in float32, out and gx in float16.  Against the oracle and against the composition on the device."""
    import chainer_amd as chx
    from chainer_amd import routines
    rng = np.random.default_rng(172)
    for shape in [(64, 6, 28, 28), (4, 5, 7, 7), (16, 8)]:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float16)
        gamma, beta = rng.uniform(0.5, 1.5, C).astype(np.float32), rng.standard_normal(C).astype(np.float32)
        rm0, rv0 = rng.standard_normal(C).astype(np.float32), rng.uniform(0.5, 1.5, C).astype(np.float32)
        gout = rng.standard_normal(shape).astype(np.float16)
        axis = (0,) if len(shape) == 2 else None
        res = {}
        for mode in ('kernel', 'composition'):
            routines.COMPOSE_BATCH_NORM = mode == 'composition'
            try:
                RM, RV = chx.array(rm0), chx.array(rv0)
                out, state = chx.batch_norm(chx.array(x), chx.array(gamma), chx.array(beta), RM, RV, 2e-5, 0.9, axis)
                gx, gg, gb = chx.batch_norm_grad(chx.array(x), chx.array(gamma), chx.array(gout), state, axis)
                res[mode] = [out.get(), RM.get(), RV.get(), state[0].get(), state[1].get(), gx.get(), gg.get(), gb.get()]
            finally:
                routines.COMPOSE_BATCH_NORM = False
        o_ref, rm_ref, rv_ref, st_ref = O.batch_norm(x, gamma, beta, rm0.copy(), rv0.copy(), 2e-5, 0.9, axis)
        gx_ref, gg_ref, gb_ref = O.batch_norm_grad(x, gamma, gout, st_ref, axis)
        ref = [o_ref, rm_ref, rv_ref, st_ref[0], st_ref[1], gx_ref, gg_ref, gb_ref]
        names = ['out', 'running_mean', 'running_var', 'mean', 'inv_std', 'gx', 'ggamma', 'gbeta']
        dtypes = ['float16', 'float32', 'float32', 'float32', 'float32', 'float16', 'float32', 'float32']
        for name, dt, k, c, r in zip(names, dtypes, res['kernel'], res['composition'], ref):
            assert k.dtype == np.dtype(dt) and c.dtype == np.dtype(dt), (name, k.dtype, c.dtype)
            assert np.isfinite(k).all(), name
            tol = {'out': 2e-3, 'gx': 4e-3, 'ggamma': 2e-4, 'gbeta': 2e-4}.get(name, 2e-5)
            assert_close(k.reshape(r.shape), r, tol, 'mixed batch_norm %s %r: kernel vs oracle' % (name, shape))
            assert_close(k.reshape(r.shape), c.reshape(r.shape), tol, 'mixed batch_norm %s %r: kernel vs composition' % (name, shape))


@pytest.mark.parametrize('dt', ['float32', 'float16', 'float64'])
def test_gradients_over_n_axes_have_the_bits_of_the_composition(dt):
    """ConvGradWeight, ConvTranspose and the pooling gradients with 0, 1, 3 and 4 spatial axes (the native kernels take any number,
    conv.cc:91-160, pool.cc:97-177, 304-346; the reference's test grids): plain kernels that follow the order of the native Dot loop
    and of Col2Im's additions, so the results equal the oracle's compositions bit for bit."""
    import chainer_amd as chx
    from test_oracle_pins import CONV_ND_GRID, POOL_ND_GRID
    rng = np.random.default_rng(91)
    for xs, ws, stride, pad in CONV_ND_GRID:
        if len(xs) == 4:
            continue  # two spatial axes: the dedicated kernels, tested above
        n = len(xs) - 2
        x = rng.standard_normal(xs).astype(dt)
        w = rng.standard_normal(ws).astype(dt)
        for cv in (False, True):
            gy = rng.standard_normal(O.conv_nd(x, w, None, stride, pad, cv).shape).astype(dt)
            what = '%s %s' % (dt, (xs, ws, stride, pad, cv))
            gw = chx.conv_grad_weight(dt, ws, chx.array(x), chx.array(gy), stride, pad, cv)
            assert_exact(gw.get(), O.conv_grad_weight_nd(ws, x, gy, stride, pad, cv), 'conv_grad_weight ' + what)
            gx = chx.conv_transpose(chx.array(gy), chx.array(w), None, stride, pad, xs[2:])
            assert_exact(gx.get(), O.conv_transpose_nd(gy, w, None, stride, pad, xs[2:]), 'conv_transpose as the data gradient ' + what)
        wt = rng.standard_normal((xs[1], 4) + tuple(ws[2:])).astype(dt)
        b = rng.standard_normal(4).astype(dt)
        ref = None
        try:
            ref = O.conv_transpose_nd(x, wt, b, stride, pad)
        except ValueError:
            pass  # the default output size is not positive for this case
        if ref is not None and ref.size:
            got = chx.conv_transpose(chx.array(x), chx.array(wt), chx.array(b), stride, pad)
            assert_exact(got.get(), ref, 'conv_transpose with bias %s %s' % (dt, (xs, ws, stride, pad)))
    for xs, ks, stride, pad in POOL_ND_GRID:
        if len(xs) == 4:
            continue
        x = rng.standard_normal(xs).astype(dt)
        x.flat[::3] = x.flat[1::3][:x.flat[::3].size]  # ties inside windows: the ArgMax rule decides
        X = chx.array(x)
        for cv in (False, True):
            g = rng.standard_normal(O.max_pool_nd(x, ks, stride, pad, cv).shape).astype(dt)
            what = '%s %s' % (dt, (xs, ks, stride, pad, cv))
            assert_exact(chx.max_pool_grad(X, chx.array(g), ks, stride, pad, cv).get(), O.max_pool_grad_nd(x, g, ks, stride, pad, cv),
                         'max_pool_grad ' + what)
            gg = rng.standard_normal(xs).astype(dt)
            assert_exact(chx.max_pool_grad_grad(X, chx.array(gg), ks, stride, pad, cv).get(), O.max_pool_grad_grad_nd(x, gg, ks, stride, pad, cv),
                         'max_pool_grad_grad ' + what)
        for mode in ('zero', 'ignore'):
            g = rng.standard_normal(O.average_pool_nd(x, ks, stride, pad, mode).shape).astype(dt)
            got = chx.average_pool_grad(X, chx.array(g), ks, stride, pad, mode).get()
            ref = O.average_pool_grad_nd(x, g, ks, stride, pad, mode)
            assert np.array_equal(got, ref, equal_nan=True), 'average_pool_grad %s %s' % (dt, (xs, ks, stride, pad, mode))

"""Activations composed from other routines and the n-step recurrent family, device against the CPU oracle.

Both sides run the same sequence of kernels in the same order (the reference's composition); the only differences are the
libm-class functions (exp, tanh, log1p), so float32 agrees to 1e-5 relative and float16 to 2e-2."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close
from test_oracle_pins import _rnn_problem

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('dt', ['float32', 'float16', 'float64'])
def test_composed_activations(dt):
    import chainer_amd as chx
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((5, 8, 3)) * 3).astype(dt)
    x[0, 0, 0] = 0
    x[0, 1, 0] = np.nan
    X = chx.array(x)
    assert_close(chx.clipped_relu(X, 2.5).get(), O.clipped_relu(x, 2.5), what='clipped_relu')
    assert_close(chx.crelu(X, 1).get(), O.crelu(x, 1), what='crelu axis 1')
    assert_close(chx.crelu(X, 2).get(), O.crelu(x, 2), what='crelu axis 2')
    assert_close(chx.elu(X, 0.7).get(), O.elu(x, 0.7), what='elu')
    assert_close(chx.leaky_relu(X, 0.1).get(), O.leaky_relu(x, 0.1), what='leaky_relu')
    assert_close(chx.softplus(X, 1.7).get(), O.softplus(x, 1.7), what='softplus')
    c1, c2, c3 = rng.standard_normal((3, 6, 10)).astype(dt)
    g2 = rng.standard_normal((6, 50)).astype(dt)
    g3 = rng.standard_normal((6, 60)).astype(dt)
    for got, ref in zip(chx.tree_lstm(chx.array(c1), chx.array(c2), chx.array(g2)), O.tree_lstm(c1, c2, g2)):
        assert_close(got.get(), ref, what='tree_lstm 2-ary')
    for got, ref in zip(chx.tree_lstm(chx.array(c1), chx.array(c2), chx.array(c3), chx.array(g3)), O.tree_lstm(c1, c2, c3, g3)):
        assert_close(got.get(), ref, what='tree_lstm 3-ary')
    x1, x2 = rng.standard_normal((2, 6, 40)).astype(dt)
    for got, ref in zip(chx.slstm(chx.array(c1), chx.array(c2), chx.array(x1), chx.array(x2)), O.slstm(c1, c2, x1, x2)):
        assert_close(got.get(), ref, what='slstm')
    xi = np.arange(-3, 4, dtype=np.int32)
    assert_close(chx.elu(chx.array(xi)).get(), O.elu(xi), what='elu of integers computes in float32')


def _upload(chx, ws, bs, xs, hx, cx):
    W = [[chx.array(m) for m in layer] for layer in ws]
    B = [[chx.array(v) for v in layer] for layer in bs]
    return W, B, [chx.array(x) for x in xs], chx.array(hx), chx.array(cx)


CASES = [('lstm', 1, False, None), ('lstm', 2, False, None), ('lstm', 2, True, None), ('gru', 1, False, None), ('gru', 2, True, None),
         ('rnn', 2, False, 'tanh'), ('rnn', 1, True, 'relu'), ('rnn', 2, True, 'tanh')]


@pytest.mark.parametrize('kind,n_layers,bidirectional,activation', CASES)
def test_n_step_family_matches_oracle(kind, n_layers, bidirectional, activation):
    import chainer_amd as chx
    rng = np.random.default_rng(11)
    for in_size, units, lengths in [(4, 3, (5, 3, 3, 1)), (40, 64, (6, 6, 6, 6, 6, 6, 6, 6)), (17, 33, (4, 2))]:
        ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, kind, n_layers, bidirectional, in_size, units, lengths)
        W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
        what = '%s layers=%d bi=%s units=%d' % (kind, n_layers, bidirectional, units)
        if kind == 'lstm':
            ref = (O.n_step_bilstm if bidirectional else O.n_step_lstm)(n_layers, hx, cx, ws, bs, xs)
            for fused in (False, True):
                got = (chx.n_step_bilstm if bidirectional else chx.n_step_lstm)(n_layers, HX, CX, W, B, X, fused=fused)
                assert_close(got[0].get(), ref[0], what='hy ' + what)
                assert_close(got[1].get(), ref[1], what='cy ' + what)
                assert len(got[2]) == len(ref[2])
                for t, (y, r) in enumerate(zip(got[2], ref[2])):
                    assert_close(y.get(), r, what='ys[%d] %s fused=%s' % (t, what, fused))
            continue
        if kind == 'gru':
            ref = (O.n_step_bigru if bidirectional else O.n_step_gru)(n_layers, hx, ws, bs, xs)
            got = (chx.n_step_bigru if bidirectional else chx.n_step_gru)(n_layers, HX, W, B, X)
        else:
            ref = (O.n_step_birnn if bidirectional else O.n_step_rnn)(n_layers, hx, ws, bs, xs, activation)
            got = (chx.n_step_birnn if bidirectional else chx.n_step_rnn)(n_layers, HX, W, B, X, activation)
        assert_close(got[0].get(), ref[0], what='hy ' + what)
        assert len(got[1]) == len(ref[1])
        for t, (y, r) in enumerate(zip(got[1], ref[1])):
            assert_close(y.get(), r, what='ys[%d] %s' % (t, what))


def test_n_step_lstm_float16_and_errors():
    import chainer_amd as chx
    rng = np.random.default_rng(12)
    ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, 'lstm', 2, False, 24, 32, (5, 5, 4, 2))
    h = lambda tree: [[a.astype(np.float16) for a in layer] for layer in tree]
    ws, bs = h(ws), h(bs)
    xs = [x.astype(np.float16) for x in xs]
    hx, cx = hx.astype(np.float16), cx.astype(np.float16)
    W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
    ref = O.n_step_lstm(2, hx, cx, ws, bs, xs)
    got = chx.n_step_lstm(2, HX, CX, W, B, X)
    assert_close(got[0].get(), ref[0], what='hy float16')
    assert_close(got[1].get(), ref[1], what='cy float16')
    for y, r in zip(got[2], ref[2]):
        assert_close(y.get(), r, what='ys float16')
    with pytest.raises(chx.DimensionError):  # a batch larger than the state
        chx.n_step_lstm(2, HX[:, :3], CX[:, :3], W, B, X)


@pytest.mark.parametrize('n_layers', [1, 2, 3, 5])
def test_n_step_lstm_kernel_entry_matches_oracle(n_layers):
    """hipcx_n_step_lstm (weights packed once, one launch per wavefront stage) against the oracle's routine composition: odd sizes
    (reduction tails, partial unit and row tiles), ragged and non-monotonic step batches, more layers than one launch takes, and
    the workload's own size."""
    import chainer_amd as chx
    rng = np.random.default_rng(13 + n_layers)
    # (input size, units, sequence lengths): the batch is the number of sequences, step t holds the sequences longer than t
    problems = [(4, 3, (5, 3, 3, 1)), (40, 64, (6,) * 8), (17, 33, (4, 2)), (50, 70, (3,) * 100 + (2,) * 20 + (1,) * 10),
                (23, 9, (7,) * 66 + (2,) * 5)]
    if n_layers == 2:
        problems.append((650, 650, (2,) * 128))
    for in_size, units, lengths in problems:
        ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, 'lstm', n_layers, False, in_size, units, lengths)
        if units == 9:  # step batches that grow again (the routine only asks for batch <= state rows)
            xs = [xs[0][:5], xs[1], xs[2][:1], xs[3]]
        if units == 650:  # the workload's weight range (+-0.05): with +-0.6 the 1300-term sums reach ~12 and their rounding alone 2e-5
            ws = [[m / np.float32(12) for m in layer] for layer in ws]
        W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
        ref = O.n_step_lstm(n_layers, hx, cx, ws, bs, xs)
        got = chx.n_step_lstm(n_layers, HX, CX, W, B, X, kernel=True)
        what = 'layers=%d in=%d units=%d lengths=%r' % (n_layers, in_size, units, lengths)
        assert_close(got[0].get(), ref[0], what='hy ' + what)
        assert_close(got[1].get(), ref[1], what='cy ' + what)
        assert len(got[2]) == len(ref[2])
        for t, (y, r) in enumerate(zip(got[2], ref[2])):
            assert y.shape == r.shape
            assert_close(y.get(), r, what='ys[%d] %s' % (t, what))
        np.testing.assert_array_equal(HX.get(), hx)  # the inputs are left alone
        np.testing.assert_array_equal(CX.get(), cx)


def test_n_step_lstm_kernel_entry_special_values():
    """An inf in the initial hidden state or in an input row reaches the gates as +-inf (saturated sigmoids, tanh +-1), as in the
    routine composition -- the kernel's zero-weight blocks past the end of a row's reduction form no 0 * inf products.  Sizes whose
    reduction ends inside a chunk, so that such blocks exist."""
    import chainer_amd as chx
    rng = np.random.default_rng(77)
    for in_size, units, lengths in [(17, 33, (4, 4, 2)), (40, 70, (3,) * 20)]:
        ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, 'lstm', 1, False, in_size, units, lengths)
        ws = [[np.abs(m) + np.float32(0.01) for m in layer] for layer in ws]  # one sign: inf * w sums to inf, never inf - inf
        hx[0, 0, :3] = np.inf
        hx[0, 1, 0] = -np.inf
        xs[0][2, 1] = np.inf
        W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
        ref = O.n_step_lstm(1, hx, cx, ws, bs, xs)
        got = chx.n_step_lstm(1, HX, CX, W, B, X, kernel=True)
        what = 'in=%d units=%d' % (in_size, units)
        assert np.isfinite(ref[0]).all() and np.isfinite(ref[2][0]).all(), what  # saturated gates, finite states
        assert_close(got[0].get(), ref[0], what='hy ' + what)
        assert_close(got[1].get(), ref[1], what='cy ' + what)
        for t, (y, r) in enumerate(zip(got[2], ref[2])):
            assert_close(y.get(), r, what='ys[%d] %s' % (t, what))


def test_n_step_lstm_kernel_entry_views_and_errors():
    import ctypes
    import chainer_amd as chx
    from chainer_amd import _lib, routines
    rng = np.random.default_rng(14)
    ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, 'lstm', 2, False, 12, 20, (6, 6, 4))
    W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
    ref = O.n_step_lstm(2, hx, cx, ws, bs, xs)
    # transposed weight storage and inputs that are column slices of a wider array (rows not 16-byte aligned)
    Wt = [[chx.array(np.ascontiguousarray(m.T)).transpose((1, 0)) for m in layer] for layer in ws]
    wide = [chx.array(np.concatenate([np.zeros((x.shape[0], 1), np.float32), x], 1)) for x in xs]
    Xv = [w[:, 1:] for w in wide]
    got = chx.n_step_lstm(2, HX, CX, Wt, B, Xv, kernel=True)
    assert_close(got[0].get(), ref[0], what='hy, operands that are views')
    for y, r in zip(got[2], ref[2]):
        assert_close(y.get(), r, what='ys, operands that are views')
    with pytest.raises(chx.DimensionError):  # a batch larger than the state
        chx.n_step_lstm(2, HX[:, :2], CX[:, :2], W, B, X, kernel=True)
    with pytest.raises(chx.DimensionError):  # a weight matrix of the wrong shape
        bad = [list(layer) for layer in W]
        bad[1][2] = bad[0][0]
        chx.n_step_lstm(2, HX, CX, bad, B, X, kernel=True)
    # other dtypes are not taken by the entry: the routine composes them
    px = routines._descriptor_pointers(X)
    h16 = chx.array(hx.astype(np.float16))
    assert _lib.load().hipcx_n_step_lstm_workspace_size(2, h16.desc(), px, len(X)) == 0
    assert _lib.load().hipcx_n_step_lstm_workspace_size(2, HX.desc(), px, len(X)) > 0


def _oracle_forward(kind, n_layers, bidirectional, activation, hx, cx, ws, bs, xs):
    """(hy, cy or None, ys) of the oracle's routine composition for one family member."""
    if kind == 'lstm':
        return (O.n_step_bilstm if bidirectional else O.n_step_lstm)(n_layers, hx, cx, ws, bs, xs)
    if kind == 'gru':
        hy, ys = (O.n_step_bigru if bidirectional else O.n_step_gru)(n_layers, hx, ws, bs, xs)
    else:
        hy, ys = (O.n_step_birnn if bidirectional else O.n_step_rnn)(n_layers, hx, ws, bs, xs, activation)
    return hy, None, ys


@pytest.mark.parametrize('kind,n_layers,bidirectional,activation', CASES + [('gru', 3, False, None), ('rnn', 3, True, 'relu')])
def test_rnn_kernel_forward_matches_oracle(kind, n_layers, bidirectional, activation):
    """hipcx_n_step_rnn (RnnKernel, CX/kernels/rnn.h:34-49) in every mode and direction against the oracle's routine composition:
    inference and training (reserve kept) give the same outputs; ragged and non-monotonic step batches; odd sizes."""
    import chainer_amd as chx
    rng = np.random.default_rng(21)
    for in_size, units, lengths in [(4, 3, (5, 3, 3, 1)), (40, 64, (6,) * 8), (17, 33, (4, 2)), (23, 9, (7,) * 66 + (2,) * 5)]:
        ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, kind, n_layers, bidirectional, in_size, units, lengths)
        if units == 9 and not bidirectional:  # step batches that grow again (the routine only asks for batch <= state rows)
            xs = [xs[0][:5], xs[1], xs[2][:1], xs[3]]
        W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
        hy_ref, cy_ref, ys_ref = _oracle_forward(kind, n_layers, bidirectional, activation, hx, cx, ws, bs, xs)
        what = '%s layers=%d bi=%s act=%s in=%d units=%d' % (kind, n_layers, bidirectional, activation, in_size, units)
        for training in (False, True):
            (hy, cy), ys, state = chx.rnn(n_layers, HX, CX if kind == 'lstm' else None, W, B, X, bidirectional, kind, activation, training)
            assert (state is not None) == training
            assert_close(hy.get(), hy_ref, 2e-5, 'hy %s training=%s' % (what, training))
            if kind == 'lstm':
                assert_close(cy.get(), cy_ref, 2e-5, 'cy ' + what)
            else:
                assert cy is None
            assert len(ys) == len(ys_ref)
            for t, (y, r) in enumerate(zip(ys, ys_ref)):
                assert_close(y.get(), r, 2e-5, 'ys[%d] %s' % (t, what))
        np.testing.assert_array_equal(HX.get(), hx)  # the inputs are left alone


@pytest.mark.parametrize('kind,n_layers,bidirectional,activation', CASES)
def test_rnn_backward_kernel_matches_finite_differences(kind, n_layers, bidirectional, activation):
    """hipcx_n_step_rnn_backward (RnnBackwardKernel, CX/kernels/rnn.h:51-66) against central differences of the oracle's forward
    composition in float64: with loss = <hy, dhy> + <cy, dcy> + sum_t <ys[t], dys[t]>, every entry of dhx, dcx, dws, dbs and dxs is
    the derivative of the loss by the matching input entry.  Ragged batches (rows whose sequence has ended carry their state and its
    gradient), one dys entry and dcy absent (zeros)."""
    import chainer_amd as chx
    rng = np.random.default_rng(31 + n_layers)
    in_size, units, lengths = 4, 3, (5, 3, 3, 1)
    ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, kind, n_layers, bidirectional, in_size, units, lengths)
    if activation == 'relu':  # keep the pre-activations away from the kink, where a central difference is not the derivative
        bs = [[b + np.float32(0.5) * np.sign(b) for b in group] for group in bs]
    d = 2 if bidirectional else 1
    dhy = rng.standard_normal(hx.shape).astype(np.float32)
    dcy = rng.standard_normal(hx.shape).astype(np.float32) if n_layers == 1 else None
    dys = [rng.standard_normal((x.shape[0], d * units)).astype(np.float32) for x in xs]
    dys[1] = None
    W, B, X, HX, CX = _upload(chx, ws, bs, xs, hx, cx)
    _, _, state = chx.rnn(n_layers, HX, CX if kind == 'lstm' else None, W, B, X, bidirectional, kind, activation, True)
    (dhx, dcx), dws, dbs, dxs = chx.rnn_backward(state, chx.array(dhy), chx.array(dcy) if dcy is not None else None,
                                                 [chx.array(g) if g is not None else None for g in dys])

    f64 = lambda a: np.asarray(a, np.float64)
    p_hx, p_cx = f64(hx), f64(cx)
    p_ws, p_bs = [[f64(m) for m in g] for g in ws], [[f64(v) for v in g] for g in bs]
    p_xs = [f64(x) for x in xs]

    def loss():
        hy, cy, ys = _oracle_forward(kind, n_layers, bidirectional, activation, p_hx, p_cx, p_ws, p_bs, p_xs)
        total = float((hy * dhy).sum())
        if kind == 'lstm' and dcy is not None:
            total += float((cy * dcy).sum())
        return total + sum(float((y * g).sum()) for y, g in zip(ys, dys) if g is not None)

    def numeric(a):
        g = np.zeros(a.shape)
        eps = 1e-6
        for i in np.ndindex(*a.shape):
            keep = a[i]
            a[i] = keep + eps
            up = loss()
            a[i] = keep - eps
            down = loss()
            a[i] = keep
            g[i] = (up - down) / (2 * eps)
        return g

    what = '%s layers=%d bi=%s act=%s' % (kind, n_layers, bidirectional, activation)

    def check(got, want, name):
        got = got.get().astype(np.float64)
        assert got.shape == want.shape, name
        scale = max(np.abs(want).max(), 1.0)
        assert np.abs(got - want).max() <= 2e-4 * scale, '%s %s: max error %.3g (scale %.3g)' % (name, what, np.abs(got - want).max(), scale)

    check(dhx, numeric(p_hx), 'dhx')
    if kind == 'lstm':
        check(dcx, numeric(p_cx), 'dcx')
    else:
        assert dcx is None
    flat_w = [m for g in p_ws for m in g]
    flat_b = [v for g in p_bs for v in g]
    assert len(dws) == len(flat_w) and len(dbs) == len(flat_b)
    for i, (g, a) in enumerate(zip(dws, flat_w)):
        check(g, numeric(a), 'dws[%d]' % i)
    for i, (g, a) in enumerate(zip(dbs, flat_b)):
        check(g, numeric(a), 'dbs[%d]' % i)
    for t, (g, a) in enumerate(zip(dxs, p_xs)):
        check(g, numeric(a), 'dxs[%d]' % t)

"""Solve / Inverse / Cholesky / Eigh / Qr / Svd / Pinv against the CPU oracle (LAPACK through numpy, as the native backend calls it).

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


@pytest.mark.parametrize('dt,tol', [('float32', 1e-4), ('float64', 1e-11)])
def test_blocked_factorisations_at_block_edges_and_many_columns(dt, tol):
    """Sizes around the 32-wide block columns and the 64-wide column strips, more right-hand sides than one strip holds, and
    matrices whose panels need several rows per thread (above 1024 and above 2048 rows)."""
    import chainer_amd as chx
    rng = np.random.default_rng(11)
    for n, m in ((31, 3), (32, 64), (33, 65), (63, 1), (64, 130), (65, 7), (96, 200), (257, 5), (1100, 9), (2100, 2)):
        a = (rng.standard_normal((n, n)) + 3 * np.sqrt(n) * np.eye(n)).astype(dt)  # singular values stay well away from zero
        a = a[rng.permutation(n)]  # every column's pivot sits somewhere else
        b = rng.standard_normal((n, m)).astype(dt)
        x = chx.solve(chx.array(a), chx.array(b)).get()
        assert_close(x, O.solve(a, b), tol * n, 'solve n=%d m=%d' % (n, m))
        assert np.abs(a.astype(np.float64) @ x.astype(np.float64) - b).max() <= tol * n
        if n <= 1100:
            inv = chx.inv(chx.array(a)).get()
            assert_close(inv, O.inv(a), tol * n, 'inv n=%d' % n)
        spd = (a.astype(np.float64) @ a.T.astype(np.float64)).astype(dt)
        low = chx.cholesky(chx.array(spd)).get()
        assert_close(low, O.cholesky(spd), tol * n, 'cholesky n=%d' % n)
        assert np.array_equal(low, np.tril(low))


def test_pivot_choice_among_equal_magnitudes_and_late_failures():
    """Columns with several entries of the same largest magnitude (the first one in the current row order is the pivot, as
    LAPACK's idamax picks it), a matrix that becomes singular only in a later block column, and a Cholesky input that stops
    being positive definite there: the flag carries LAPACK's 1-based position."""
    import chainer_amd as chx
    rng = np.random.default_rng(12)
    n = 70
    a = rng.integers(-2, 3, (n, n)).astype('float64') + 3 * np.eye(n)
    b = rng.standard_normal((n, 2))
    assert_close(chx.solve(chx.array(a), chx.array(b)).get(), O.solve(a, b), 1e-9, 'integer-valued matrix')
    sing = (rng.standard_normal((n, n)) + 8 * np.eye(n)).astype('float64')
    sing[:, 50] = 0  # a zero column stays zero under elimination: the first zero pivot is at position 51
    with pytest.raises(chx.ChainerxError, match='Info = 51'):
        chx.solve(chx.array(sing), chx.array(b))
    with pytest.raises(chx.ChainerxError, match='Info = 51'):
        chx.inv(chx.array(sing))
    spd = np.eye(n) * 4.0
    spd[40, 40] = -1.0
    with pytest.raises(chx.ChainerxError, match='Info = 41'):
        chx.cholesky(chx.array(spd))


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


@pytest.mark.parametrize('dt,tol', [('float32', 2e-5), ('float64', 1e-12)])
def test_eigh(dt, tol):
    """Eigenvalues against the oracle's (LAPACK syevd); eigenvectors through what defines them (a @ v = v * w, orthonormal
    columns) and, for well separated spectra, against the oracle's up to the sign of each column -- the comparison the reference's
    own test makes (tests/chainerx_tests/unit_tests/routines_tests/test_linalg.py:510-539)."""
    import chainer_amd as chx
    rng = np.random.default_rng(4)
    for n in (1, 2, 3, 8, 33, 64, 129, 200):
        a = rng.standard_normal((n, n)).astype(dt)
        a = ((a + a.T) / 2 + 1e-3 * np.eye(n)).astype(dt)
        scale = max(np.abs(a).max() * n ** 0.5, 1.0)
        for uplo in ('u', 'L'):
            noise = rng.standard_normal((n, n)).astype(dt)
            spoiled = np.triu(a) + np.tril(noise, -1) if uplo.upper() == 'U' else np.tril(a) + np.triu(noise, 1)
            w, v = chx.eigh(chx.array(spoiled), uplo)
            assert w.shape == (n,) and v.shape == (n, n) and w.dtype == np.dtype(dt) and v.dtype == np.dtype(dt)
            w, v = w.get(), v.get()
            w_ref, v_ref = O.eigh(a, uplo)
            assert np.all(np.diff(w) >= 0), 'ascending order'
            assert np.abs(w - w_ref).max() <= tol * scale * n ** 0.5, 'eigenvalues n=%d' % n
            a64, v64 = a.astype(np.float64), v.astype(np.float64)
            assert np.abs(a64 @ v64 - v64 * w).max() <= tol * scale * n ** 0.5, 'a v = v w, n=%d' % n
            assert np.abs(v64.T @ v64 - np.eye(n)).max() <= tol * n, 'orthonormal n=%d' % n
            only_w = chx.eigvalsh(chx.array(spoiled), uplo).get()
            assert np.array_equal(only_w, w)
    # a prescribed, well separated spectrum: eigenvectors agree with LAPACK's up to sign
    n = 12
    q, _ = np.linalg.qr(rng.standard_normal((n, n)))
    d = np.arange(1, n + 1, dtype=np.float64)
    a = ((q * d) @ q.T)
    a = ((a + a.T) / 2).astype(dt)
    w, v = chx.eigh(chx.array(a))
    w_ref, v_ref = O.eigh(a)
    assert_close(w.get(), w_ref, tol * 100, 'prescribed spectrum')
    assert np.abs(np.abs(v.get()) - np.abs(v_ref)).max() <= tol * 1000
    # a transposed view and a diagonal matrix (no rotation at all: the values are only sorted)
    wt = chx.eigvalsh(chx.array(a).T, 'U').get()
    assert_close(wt, w_ref, tol * 100, 'transposed view reads the other triangle of the same symmetric matrix')
    dg = np.diag(np.array([3., -1., 2., -1.], dt))
    w, v = chx.eigh(chx.array(dg))
    assert np.array_equal(w.get(), np.array([-1., -1., 2., 3.], dt))
    assert np.array_equal(np.abs(v.get()), np.eye(4, dtype=dt)[:, [1, 3, 2, 0]])


def test_eigh_errors_and_empty():
    import chainer_amd as chx
    w, v = chx.eigh(chx.zeros((0, 0), 'float32'))
    assert w.shape == (0,) and v.shape == (0, 0)
    with pytest.raises(chx.DimensionError):
        chx.eigh(chx.zeros((2, 3), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.eigvalsh(chx.zeros((2, 2, 2), 'float32'))
    with pytest.raises(chx.DtypeError):
        chx.eigh(chx.zeros((2, 2), 'float16'))
    with pytest.raises(chx.DtypeError):
        chx.eigh(chx.zeros((2, 2), 'int32'))
    with pytest.raises(chx.ChainerxError):
        chx.eigh(chx.zeros((2, 2), 'float32'), 'X')
    with pytest.raises(TypeError):
        chx.eigh(chx.zeros((2, 2), 'float32'), None)


@pytest.mark.parametrize('dt,tol', [('float32', 2e-5), ('float64', 1e-12)])
def test_qr(dt, tol):
    """Every mode against the oracle (LAPACK geqrf / orgqr): the reflector convention is LAPACK's, so values agree including signs;
    plus the defining identities against float64."""
    import chainer_amd as chx
    rng = np.random.default_rng(5)
    for m, n in ((1, 1), (2, 2), (5, 5), (7, 3), (3, 7), (1, 6), (6, 1), (64, 64), (130, 70), (70, 130), (300, 200)):
        a = rng.standard_normal((m, n)).astype(dt)
        k = min(m, n)
        bound = tol * max(m, n)
        q, r = chx.qr(chx.array(a))
        q_ref, r_ref = O.qr(a)
        assert q.shape == q_ref.shape and r.shape == r_ref.shape and q.dtype == np.dtype(dt) and r.dtype == np.dtype(dt)
        q, r = q.get(), r.get()
        assert np.array_equal(r, np.triu(r))
        assert np.abs(q.astype(np.float64) @ r - a).max() <= bound, 'q r = a for %r' % ((m, n),)
        assert np.abs(q.T.astype(np.float64) @ q - np.eye(k)).max() <= bound
        assert np.abs(q - q_ref).max() <= bound * 10 and np.abs(r - r_ref).max() <= bound * 10, 'values and signs %r' % ((m, n),)
        qc, rc = chx.qr(chx.array(a), 'complete')
        qc_ref, rc_ref = O.qr(a, 'complete')
        assert qc.shape == (m, m) and rc.shape == (m, n)
        qc, rc = qc.get(), rc.get()
        assert np.abs(qc.astype(np.float64) @ rc - a).max() <= bound
        assert np.abs(qc.T.astype(np.float64) @ qc - np.eye(m)).max() <= bound
        assert np.abs(qc - qc_ref).max() <= bound * 10 and np.abs(rc - rc_ref).max() <= bound * 10
        assert np.abs(chx.qr(chx.array(a), 'r').get() - r_ref).max() <= bound * 10
        h, tau = chx.qr(chx.array(a), 'raw')
        h_ref, tau_ref = O.qr(a, 'raw')
        assert h.shape == (n, m) and tau.shape == (k,)
        assert np.abs(h.get() - h_ref).max() <= bound * 10 and np.abs(tau.get() - tau_ref).max() <= bound * 10
    # a transposed view; columns that are already zero below the diagonal (tau = 0, no reflection)
    a = rng.standard_normal((6, 4)).astype(dt)
    q, r = chx.qr(chx.array(a).T)
    q_ref, r_ref = O.qr(a.T)
    assert_close(q.get(), q_ref, tol * 100, 'transposed view q')
    assert_close(r.get(), r_ref, tol * 100, 'transposed view r')
    tri = np.triu(rng.standard_normal((5, 5))).astype(dt)
    q, r = chx.qr(chx.array(tri))
    assert np.array_equal(q.get(), np.eye(5, dtype=dt)) and np.array_equal(r.get(), tri)


def test_qr_errors_and_empty():
    import chainer_amd as chx
    for shape in ((0, 0), (0, 3), (3, 0)):
        for mode in ('reduced', 'complete', 'r', 'raw'):
            ref = O.qr(np.zeros(shape, 'float32'), mode)
            got = chx.qr(chx.zeros(shape, 'float32'), mode)
            ref = ref if isinstance(ref, tuple) else (ref,)
            got = got if isinstance(got, tuple) else (got,)
            for g, e in zip(got, ref):
                assert g.shape == e.shape and np.array_equal(g.get(), e), (shape, mode)
    with pytest.raises(ValueError):
        chx.qr(chx.zeros((2, 2), 'float32'), 'full')
    with pytest.raises(chx.DimensionError):
        chx.qr(chx.zeros((2, 2, 2), 'float32'))
    with pytest.raises(chx.DtypeError):
        chx.qr(chx.zeros((2, 2), 'float16'))
    with pytest.raises(chx.DtypeError):
        chx.qr(chx.zeros((2, 2), 'int32'))


@pytest.mark.parametrize('dt,tol', [('float32', 2e-5), ('float64', 1e-12)])
def test_svd_pinv(dt, tol):
    """Singular values against the oracle's (LAPACK gesdd); the factors through what defines them (reconstruction, orthonormal
    columns / rows in every shape, full and reduced) and, for a well separated spectrum, against the oracle's up to the common sign
    of u[:, i] and vt[i, :]; pinv against the oracle and the Moore-Penrose conditions."""
    import chainer_amd as chx
    rng = np.random.default_rng(6)
    for m, n in ((1, 1), (2, 2), (5, 5), (7, 3), (3, 7), (1, 6), (6, 1), (64, 64), (130, 40), (40, 130), (200, 150)):
        a = rng.standard_normal((m, n)).astype(dt)
        k = min(m, n)
        bound = tol * max(m, n)
        s_ref = O.svd(a, compute_uv=False)
        s_only = chx.svd(chx.array(a), compute_uv=False)
        assert s_only.shape == (k,) and s_only.dtype == np.dtype(dt)
        assert np.abs(s_only.get() - s_ref).max() <= bound * 4, 'singular values %r' % ((m, n),)
        for full in (True, False):
            u, s, vt = chx.svd(chx.array(a), full_matrices=full)
            assert u.shape == (m, m if full else k) and s.shape == (k,) and vt.shape == (n if full else k, n)
            u, s, vt = u.get().astype(np.float64), s.get(), vt.get().astype(np.float64)
            assert np.array_equal(s, s_only.get()) and np.all(np.diff(s) <= 0)
            assert np.abs((u[:, :k] * s) @ vt[:k] - a).max() <= bound * 4, 'u s vt = a %r full=%r' % ((m, n), full)
            assert np.abs(u.T @ u - np.eye(u.shape[1])).max() <= bound * 4, 'u orthonormal %r full=%r' % ((m, n), full)
            assert np.abs(vt @ vt.T - np.eye(vt.shape[0])).max() <= bound * 4, 'vt orthonormal %r full=%r' % ((m, n), full)
        p = chx.pinv(chx.array(a))
        assert p.shape == (n, m) and p.dtype == np.dtype(dt)
        cond = s_ref[0] / s_ref[-1]
        assert np.abs(p.get() - O.pinv(a)).max() <= bound * 10 * cond / s_ref[-1], 'pinv %r' % ((m, n),)
    # a prescribed, well separated spectrum: vectors agree with LAPACK's up to sign; a transposed view gives the transposed factors
    m, n, k = 9, 6, 6
    qu, _ = np.linalg.qr(rng.standard_normal((m, m)))
    qv, _ = np.linalg.qr(rng.standard_normal((n, n)))
    d = np.arange(k, 0, -1).astype(np.float64)
    a = ((qu[:, :k] * d) @ qv.T).astype(dt)
    u, s, vt = chx.svd(chx.array(a), full_matrices=False)
    u_ref, s_ref, vt_ref = O.svd(a, full_matrices=False)
    assert_close(s.get(), s_ref, tol * 100, 'prescribed spectrum')
    sign = np.sign((u.get() * u_ref).sum(0))
    assert np.abs(u.get() * sign - u_ref).max() <= tol * 1000 and np.abs(vt.get() * sign[:, None] - vt_ref).max() <= tol * 1000
    ut, st, vtt = chx.svd(chx.array(a).T, full_matrices=False)
    assert_close(st.get(), s_ref, tol * 100, 'transposed view')
    assert np.abs((ut.get().astype(np.float64) * st.get()) @ vtt.get() - a.T).max() <= tol * 100
    # rank deficiency: zero singular values, and the factors still orthonormal (their columns come from the completion)
    low = (rng.standard_normal((8, 2)) @ rng.standard_normal((2, 5))).astype(dt)
    low[:, 4] = 0
    for mat in (low, low.T.copy(), np.zeros((4, 3), dt)):
        u, s, vt = chx.svd(chx.array(mat))
        u, s, vt = u.get().astype(np.float64), s.get(), vt.get().astype(np.float64)
        kk = min(mat.shape)
        assert np.abs(s - O.svd(mat, compute_uv=False)).max() <= tol * 100
        assert np.abs((u[:, :kk] * s) @ vt[:kk] - mat).max() <= tol * 100
        assert np.abs(u.T @ u - np.eye(u.shape[0])).max() <= tol * 100 and np.abs(vt @ vt.T - np.eye(vt.shape[0])).max() <= tol * 100
    # pinv drops what rcond says
    dg = np.diag(np.array([2., 1e-3, 4.], dt))
    assert_close(chx.pinv(chx.array(dg), rcond=1e-2).get(), O.pinv(dg, rcond=1e-2), tol * 10, 'pinv rcond')


def test_svd_errors_and_empty():
    import chainer_amd as chx
    for shape in ((0, 0), (0, 3), (3, 0)):
        for full in (True, False):
            ref = O.svd(np.zeros(shape, 'float32'), full_matrices=full)
            got = chx.svd(chx.zeros(shape, 'float32'), full_matrices=full)
            for g, e in zip(got, ref):
                assert g.shape == e.shape and np.array_equal(g.get(), e), (shape, full)
        assert chx.svd(chx.zeros(shape, 'float32'), compute_uv=False).shape == (0,)
        assert chx.pinv(chx.zeros(shape, 'float32')).shape == shape[::-1]
    with pytest.raises(chx.DimensionError):
        chx.svd(chx.zeros((2, 2, 2), 'float32'))
    with pytest.raises(chx.DimensionError):
        chx.pinv(chx.zeros((2,), 'float32'))
    with pytest.raises(chx.DtypeError):
        chx.svd(chx.zeros((2, 2), 'float16'))
    with pytest.raises(chx.DtypeError):
        chx.pinv(chx.zeros((2, 2), 'int64'))


def test_decompositions_spread_over_workgroups_at_larger_sizes():
    """eigh, qr and svd at sizes where their sweeps / column steps run as many launches over many workgroups (odd sizes: the
    round-robin pairing has a dummy player; more columns than one strip; a matrix above 1024 rows), float32, through what
    defines the factors and against the oracle's values."""
    import chainer_amd as chx
    rng = np.random.default_rng(21)
    tol = 1e-4
    n = 513
    a = rng.standard_normal((n, n)).astype('float32')
    a = ((a + a.T) / 2).astype('float32')
    w, v = chx.eigh(chx.array(a))
    w, v = w.get(), v.get().astype(np.float64)
    scale = np.abs(a).max() * n ** 0.5
    assert np.all(np.diff(w) >= 0)
    assert np.abs(w - O.eigh(a)[0]).max() <= tol * scale * n ** 0.5
    assert np.abs(a.astype(np.float64) @ v - v * w).max() <= tol * scale * n ** 0.5
    assert np.abs(v.T @ v - np.eye(n)).max() <= tol * n
    for m, n in ((1030, 333), (333, 1030)):
        a = rng.standard_normal((m, n)).astype('float32')
        k = min(m, n)
        q, r = chx.qr(chx.array(a))
        q, r = q.get().astype(np.float64), r.get().astype(np.float64)
        assert q.shape == (m, k) and r.shape == (k, n)
        assert np.abs(q @ r - a).max() <= tol * max(m, n) and np.abs(q.T @ q - np.eye(k)).max() <= tol * max(m, n)
        assert np.array_equal(r, np.triu(r))
        q_ref, r_ref = O.qr(a)
        assert np.abs(np.abs(np.diag(r)) - np.abs(np.diag(r_ref))).max() <= tol * max(m, n)
        u, sv, vt = chx.svd(chx.array(a), full_matrices=False)
        u, sv, vt = u.get().astype(np.float64), sv.get(), vt.get().astype(np.float64)
        assert np.abs(sv - O.svd(a, compute_uv=False)).max() <= tol * max(m, n) * 4
        assert np.abs((u * sv) @ vt - a).max() <= tol * max(m, n) * 4
        assert np.abs(u.T @ u - np.eye(k)).max() <= tol * max(m, n) * 4 and np.abs(vt @ vt.T - np.eye(k)).max() <= tol * max(m, n) * 4
    # svd of matrices whose column-block pairs do not fit into LDS (the rotations then run on the columns in memory), a short last
    # block of columns and an odd number of blocks; wide input (the transposed problem) and singular values only as well
    for dt, (m, n), rtol in (('float32', (1300, 70), 1e-4), ('float64', (700, 90), 1e-12), ('float64', (90, 700), 1e-12)):
        a = rng.standard_normal((m, n)).astype(dt)
        k = min(m, n)
        u, sv, vt = chx.svd(chx.array(a), full_matrices=False)
        u, sv, vt = u.get().astype(np.float64), sv.get().astype(np.float64), vt.get().astype(np.float64)
        bound = rtol * max(m, n) * 4
        assert np.abs(sv - O.svd(a, compute_uv=False)).max() <= bound and np.all(np.diff(sv) <= 0)
        assert np.abs((u * sv) @ vt - a).max() <= bound
        assert np.abs(u.T @ u - np.eye(k)).max() <= bound and np.abs(vt @ vt.T - np.eye(k)).max() <= bound
        only = chx.svd(chx.array(a), compute_uv=False)
        only = only[1] if isinstance(only, (tuple, list)) else only
        assert np.abs(only.get().astype(np.float64) - sv).max() <= bound


def test_eigh_above_one_workgroup_on_hard_spectra():
    """eigh above 64 rows runs the SVD's one-sided block sweeps on A + |A|_F I and takes the eigenvalues as Rayleigh quotients:
    spectra that would defeat one-sided rotations without the shift (pairs +-lambda, repeated and zero eigenvalues, a matrix
    whose columns are orthogonal as they stand), through what defines an eigendecomposition.
    Bar: 20 eps sqrt(n) |A|_2 for eigenvalues, 40 eps sqrt(n) |A|_2 for residuals, 20 eps n for orthogonality."""
    import chainer_amd as chx
    rng = np.random.default_rng(22)
    for dt, eps in (('float32', 1.2e-7), ('float64', 2.3e-16)):
        n = 200
        q, _ = np.linalg.qr(rng.standard_normal((n, n)))
        half = np.logspace(-6, 0, n // 2)
        cases = {
            'random': (lambda g: (g + g.T) / 2)(rng.standard_normal((333, 333))),
            'pairs': (q * np.concatenate([half, -half])) @ q.T,
            'repeated': (q * np.repeat([1.0, -1.0, 0.5, 0.0], n // 4)) @ q.T,
            'antidiagonal': np.fliplr(np.eye(96)),  # eigenvalues +-1 only
            'zero': np.zeros((70, 70)),
        }
        if dt == 'float64':  # too many rows for the block pairs to sit in LDS: the sweeps rotate the columns in memory
            cases['random, in memory'] = (lambda g: (g + g.T) / 2)(rng.standard_normal((600, 600)))
        for name, a in cases.items():
            a = ((a + a.T) / 2).astype(dt)
            m = a.shape[0]
            w, v = chx.eigh(chx.array(a))
            w, v = w.get().astype(np.float64), v.get().astype(np.float64)
            a64 = a.astype(np.float64)
            scale = eps * np.sqrt(m) * max(np.abs(np.linalg.eigvalsh(a64)).max(), 0.0)
            assert np.all(np.diff(w) >= 0), (dt, name)
            assert np.abs(w - np.linalg.eigvalsh(a64)).max() <= 20 * scale, (dt, name)
            assert np.abs(a64 @ v - v * w).max() <= 40 * scale, (dt, name)
            assert np.abs(v.T @ v - np.eye(m)).max() <= 20 * eps * m, (dt, name)
            only = chx.eigvalsh(chx.array(a)).get().astype(np.float64)
            assert np.abs(only - w).max() <= 20 * scale, (dt, name)


def test_one_workgroup_limits():
    """Matrices beyond what the one-workgroup kernels take are refused before anything is launched."""
    import chainer_amd as chx
    big = chx.zeros((4097, 4097), 'float32')
    with pytest.raises(chx.ChainerxNotImplementedError):
        chx.eigh(big)
    with pytest.raises(chx.ChainerxNotImplementedError):
        chx.svd(big)



def test_svd_and_eigh_are_captured_into_a_graph_without_host_waits():
    """Above one workgroup's size the Jacobi sweeps are separate launches that end when a sweep rotates nothing.  Outside capture the
    host reads that flag; on a capturing stream (where it cannot) a fixed number of sweeps is recorded, each gated on the flag of the
    sweep before it.  Both run the same rotations: the replays equal the eager results bit for bit, also after the input changed."""
    import torch
    import chainer_amd as chx
    from chainer_amd import routines
    from chainer_amd.graph import capture
    rng = np.random.default_rng(77)
    n = 150
    a0 = rng.standard_normal((n, n)).astype(np.float32)
    a1 = (rng.standard_normal((n, n)) * np.linspace(1e-3, 1.0, n)).astype(np.float32)  # graded columns: more sweeps
    A = chx.array(a0)
    S = chx.array(((a0 + a0.T) / 2).astype(np.float32))
    g_svd = capture(lambda: chx.svd(A, full_matrices=False))
    g_eig = capture(lambda: chx.eigh(S))
    for a in (a0, a1, np.zeros((n, n), np.float32), a0):
        sym = ((a + a.T) / 2).astype(np.float32)
        routines._copy_into(A, chx.array(a))  # new values in the buffers the graphs read
        routines._copy_into(S, chx.array(sym))
        u, s, vt = (t.get() for t in chx.svd(A, full_matrices=False))
        w, v = (t.get() for t in chx.eigh(S))
        g_svd.replay()
        g_eig.replay()
        torch.cuda.synchronize()
        ur, sr, vtr = (t.get() for t in g_svd.result)
        wr, vr = (t.get() for t in g_eig.result)
        assert np.array_equal(sr, s) and np.array_equal(ur, u) and np.array_equal(vtr, vt)
        assert np.array_equal(wr, w) and np.array_equal(vr, v)
        if a.any():
            assert np.abs((ur.astype(np.float64) * sr) @ vtr - a).max() <= 1e-4 * np.abs(a).max() * n
            assert np.abs(sym.astype(np.float64) @ vr - vr.astype(np.float64) * wr).max() <= 1e-4 * np.abs(sym).max() * n
    g_svd.release()
    g_eig.release()

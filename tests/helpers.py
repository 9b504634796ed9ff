"""Shared test helpers: padded (non-contiguous) arrays like the reference's testing::BuildArray(...).WithPadding(n)
(CX/testing/array.h:53-141), uploads that keep a numpy view's strides, and tolerance checks."""
import numpy as np


def padded(shape, data=None, padding=1, dtype=np.float32, start=0, step=1):
    """numpy view with BuildArray's stride rule: innermost first, `st += itemsize * pad; strides[i] = st; st *= shape[i]`.
    `data` None -> WithLinearData(start, step)."""
    dtype = np.dtype(dtype)
    shape = tuple(shape)
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    if data is None:
        data = start + step * np.arange(n)
    vals = np.asarray(data).astype(dtype).reshape(shape)
    pads = (padding,) * len(shape) if isinstance(padding, int) else tuple(padding)
    strides = [0] * len(shape)
    st = dtype.itemsize
    for i in reversed(range(len(shape))):
        st += dtype.itemsize * pads[i]
        strides[i] = st
        st *= shape[i]
    buf = np.full(max(st, dtype.itemsize), 0xff, np.uint8)
    view = np.ndarray(shape, dtype, buffer=buf, offset=0, strides=strides)
    view[...] = vals
    return view


def upload_view(chx, view):
    """Uploads the bytes a numpy view spans and returns a device array with the same shape and (byte) strides."""
    import ctypes
    view = np.asarray(view)
    if view.size == 0:
        return chx.ndarray.empty(view.shape, view.dtype)
    lo = sum((d - 1) * s for d, s in zip(view.shape, view.strides) if s < 0)
    hi = sum((d - 1) * s for d, s in zip(view.shape, view.strides) if s > 0) + view.dtype.itemsize
    addr = view.__array_interface__['data'][0] + lo
    raw = np.frombuffer((ctypes.c_ubyte * (hi - lo)).from_address(addr), np.uint8).copy()
    dev = chx.array(raw)
    return chx.ndarray(dev._buf, -lo, view.shape, view.strides, view.dtype)


def channels_last(chx, x):
    """Device array with NCHW shape over NHWC memory."""
    nhwc = np.ascontiguousarray(x.transpose(0, 2, 3, 1))
    return chx.array(nhwc).transpose(0, 3, 1, 2)


# Tolerances of the parity contract: 1e-5 relative for float32, 2e-2 for float16 (after fp32 accumulation); float64 is
# held to 1e-12.  Two readings of "relative" are checked:
#   * tensor-relative (always): max |got - ref| / max |ref| <= rtol, so that entries that cancel to ~0 are judged on the
#     scale of the tensor they belong to;
#   * element-wise (with elementwise=True; the five workload tests use it): |got - ref| <= rtol * |ref| + atol * max |ref|
#     for every element, with the absolute terms the reference's own operator tests pair their rtol with: 5e-3 for float16
#     (tests/chainerx_tests/unit_tests/routines_tests/test_connection.py:124-126) and 1e-5 for float32
#     (test_normalization.py:136-138), taken relative to the output's scale (the reference's tests draw O(1) data).
RTOL = {np.dtype('float16'): 2e-2, np.dtype('float32'): 1e-5, np.dtype('float64'): 1e-12}
ATOL = {np.dtype('float16'): 5e-3, np.dtype('float32'): 1e-5, np.dtype('float64'): 1e-12}


def error_figures(got, ref):
    """(tensor-relative error, largest element-wise relative error over elements above 1e-3 of the scale)."""
    g = np.asarray(got).astype(np.float64)
    r = np.asarray(ref).astype(np.float64)
    fin = np.isfinite(r)
    if not fin.any():
        return 0.0, 0.0
    scale = max(np.abs(r[fin]).max(), 1e-30)
    diff = np.abs(g[fin] - r[fin])
    big = np.abs(r[fin]) > 1e-3 * scale
    return float(diff.max() / scale), float((diff[big] / np.abs(r[fin][big])).max()) if big.any() else 0.0


def assert_close(got, ref, rtol=None, what='', elementwise=False):
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape, '%s: shape %r != %r' % (what, got.shape, ref.shape)
    assert got.dtype == ref.dtype, '%s: dtype %s != %s' % (what, got.dtype, ref.dtype)
    if rtol is None:
        rtol = RTOL[ref.dtype]
    g = got.astype(np.float64)
    r = ref.astype(np.float64)
    nan_g, nan_r = np.isnan(g), np.isnan(r)
    assert np.array_equal(nan_g, nan_r), '%s: NaN pattern differs' % what
    inf = np.isinf(r)
    assert np.array_equal(g[inf], r[inf]), '%s: infinities differ' % what
    fin = ~(nan_r | inf)
    if not fin.any():
        return
    scale = max(np.abs(r[fin]).max(), 1e-30)
    err = np.abs(g[fin] - r[fin]).max() / scale
    assert err <= rtol, '%s: max |got-ref| / max|ref| = %.3g > %.3g' % (what, err, rtol)
    if elementwise:
        atol = ATOL.get(ref.dtype, 0.0) * scale
        excess = np.abs(g[fin] - r[fin]) - (rtol * np.abs(r[fin]) + atol)
        worst = int(np.argmax(excess))
        assert excess[worst] <= 0, '%s: element-wise |got-ref| <= %.3g |ref| + %.3g fails: got %r, ref %r' % (
            what, rtol, atol, g[fin][worst], r[fin][worst])
        tensor_rel, elem_rel = error_figures(got, ref)
        print('%s: tensor-relative error %.3g, largest element-wise relative error %.3g (rtol %.3g, atol %.3g of the scale)' % (
            what or 'assert_close', tensor_rel, elem_rel, rtol, ATOL.get(ref.dtype, 0.0)))


def assert_exact(got, ref, what=''):
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape, '%s: shape %r != %r' % (what, got.shape, ref.shape)
    assert got.dtype == ref.dtype, '%s: dtype %s != %s' % (what, got.dtype, ref.dtype)
    if got.dtype.kind == 'f':
        same = (got.view(np.dtype('u%d' % got.dtype.itemsize)) == ref.view(np.dtype('u%d' % ref.dtype.itemsize))) | (np.isnan(got) & np.isnan(ref))
        assert same.all(), '%s: %d of %d elements differ bitwise' % (what, int((~same).sum()), same.size)
    else:
        assert np.array_equal(got, ref), '%s: values differ' % what

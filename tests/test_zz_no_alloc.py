"""hipcx_sum_static_scratch (the entry point that allocates nothing) against hipcx_sum with a caller-provided workspace:
bit-identical results, on consecutive calls that share the library's static scratch array, the later ones smaller."""
import ctypes

import numpy as np
import pytest

from helpers import assert_exact

pytestmark = pytest.mark.gpu


def _both(chx, x, axis):
    """(hipcx_sum through the routine, hipcx_sum_static_scratch through the C ABI) for one input."""
    from chainer_amd import _lib
    from chainer_amd._array import current_stream
    X = chx.array(x)
    ref = chx.sum(X, axis=axis)
    out = chx.ndarray.empty(ref.shape, ref.dtype)
    out.fill(0)
    ax = (ctypes.c_int8 * 1)(axis)
    need = _lib.load().hipcx_reduce_workspace_size(X.desc(), ax, 1, out.desc())
    _lib.call('hipcx_sum_static_scratch', X.desc(), ax, 1, out.desc(), current_stream())
    return ref.get(), out.get(), need


def test_static_scratch_sum_matches_workspace_sum_on_consecutive_calls():
    import chainer_amd as chx
    rng = np.random.default_rng(77)
    needs = []
    # rows split over several workgroups (per-block partials), then a smaller one of the same kind, then a long strided
    # axis (per-slice partials) and a smaller one of those: each call leaves its partials behind for the next
    for shape, axis, dt in [((64, 262144), 1, 'float32'), ((16, 40000), 1, 'float32'), ((8192, 512), 0, 'float32'),
                            ((3000, 40), 0, 'float16'), ((5, 70000), 1, 'float64'), ((7, 300), 1, 'int32')]:
        x = rng.standard_normal(shape).astype(dt) if dt != 'int32' else rng.integers(-50, 50, shape).astype(dt)
        ref, got, need = _both(chx, x, axis)
        needs.append(need)
        assert_exact(got, ref, 'sum_static_scratch %r axis %d %s' % (shape, axis, dt))
    assert needs[0] > 0 and needs[1] > 0 and needs[1] < needs[0], needs   # both use the scratch, the second less of it
    assert needs[2] > 0 and needs[3] > 0, needs


def test_static_scratch_sum_refuses_reductions_beyond_its_size():
    import chainer_amd as chx
    from chainer_amd import _lib
    from chainer_amd._array import current_stream
    # many outputs x many slices of a long strided axis: more partial results than the static array holds
    X = chx.zeros((4096, 16384), 'float64')
    out = chx.ndarray.empty((16384,), 'float64')
    ax = (ctypes.c_int8 * 1)(0)
    need = _lib.load().hipcx_reduce_workspace_size(X.desc(), ax, 1, out.desc())
    if need <= (4 << 20):
        pytest.skip('this launch plan fits the static scratch (%d bytes)' % need)
    with pytest.raises(chx.ChainerxError, match='static scratch'):
        _lib.call('hipcx_sum_static_scratch', X.desc(), ax, 1, out.desc(), current_stream())


def test_static_scratch_sum_calls_on_two_streams_take_turns():
    """Calls from different streams share the one static array of the device: each waits for the previous call's kernels, so
    interleaved calls on two streams give the results of hipcx_sum."""
    import torch
    import chainer_amd as chx
    from chainer_amd import _lib
    rng = np.random.default_rng(78)
    xs = [rng.standard_normal((64, 262144)).astype('float32'), rng.standard_normal((48, 200000)).astype('float32')]
    X = [chx.array(x) for x in xs]
    refs = [chx.sum(a, axis=1).get() for a in X]
    outs = [chx.ndarray.empty((a.shape[0],), 'float32') for a in X]
    for o in outs:
        o.fill(0)
    chx.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    ax = (ctypes.c_int8 * 1)(1)
    for rep in range(6):
        for i in (0, 1):
            _lib.call('hipcx_sum_static_scratch', X[i].desc(), ax, 1, outs[i].desc(), ctypes.c_void_p(streams[i].cuda_stream))
    torch.cuda.synchronize()
    for i in (0, 1):
        assert_exact(outs[i].get(), refs[i], 'sum_static_scratch on stream %d' % i)

"""Device layer of the backend through the C ABI: pooled allocation, uploads through pinned staging, blocking read-back,
device-to-device copies, pointer checks, arenas under a HIP graph (chainerx::Device, CX/device.h:24-71, as the CUDA backend
implements it in CX/cuda/cuda_device/memory.cc)."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _lib():
    from chainer_amd import _lib
    return _lib


def _stream():
    from chainer_amd._array import current_stream
    return current_stream()


def test_malloc_free_reuse_and_stats():
    L = _lib()
    import chainer_amd as chx
    chx.synchronize()
    before = chx.pool_stats()
    p = ctypes.c_void_p()
    L.call('hipcx_malloc', 0, 0, ctypes.byref(p))
    assert p.value is None                      # Allocate(0) is a null pointer
    L.call('hipcx_malloc', 0, 1000, ctypes.byref(p))
    first = p.value
    assert first is not None and first % 256 == 0
    mid = chx.pool_stats()
    assert mid['in_use_blocks'] == before['in_use_blocks'] + 1
    assert mid['in_use_bytes'] == before['in_use_bytes'] + 1024   # rounded to the 512-byte unit's size class
    L.call('hipcx_free', 0, ctypes.c_void_p(first))
    L.call('hipcx_malloc', 0, 700, ctypes.byref(p))                # same class: the cached block
    assert p.value == first
    L.call('hipcx_free', 0, p)
    L.call('hipcx_free', 0, ctypes.c_void_p(None))                 # freeing null is fine
    with pytest.raises(chx.ChainerxError, match='out-of-pool'):
        L.call('hipcx_free', 0, ctypes.c_void_p(first + 512))
    after = chx.pool_stats()
    assert after['in_use_blocks'] == before['in_use_blocks']
    with pytest.raises(chx.DeviceError):
        L.call('hipcx_malloc', 63, 16, ctypes.byref(p))


def test_out_of_memory_is_reported_after_releasing_the_cache():
    L = _lib()
    import chainer_amd as chx
    p = ctypes.c_void_p()
    L.call('hipcx_malloc', 0, 64 << 20, ctypes.byref(p))
    L.call('hipcx_free', 0, p)
    assert chx.pool_stats()['cached_bytes'] >= 64 << 20
    with pytest.raises(chx.OutOfMemoryError, match='Out of memory allocating'):
        L.call('hipcx_malloc', 0, 1 << 45, ctypes.byref(p))       # 32 TiB: the driver refuses, twice
    assert chx.pool_stats()['cached_bytes'] == 0                   # the retry released the general cache
    x = chx.array(np.arange(10, dtype=np.float32))                 # and the pool still works
    assert np.array_equal((x + x).get(), 2 * np.arange(10, dtype=np.float32))


@pytest.mark.parametrize('nbytes', [1, 513, 4096 + 17, (3 << 20) + 5])
def test_host_round_trip_and_device_copy(nbytes):
    L = _lib()
    rng = np.random.default_rng(nbytes)
    src = rng.integers(0, 256, nbytes, dtype=np.uint8)
    dev = ctypes.c_void_p()
    L.call('hipcx_from_host_memory', 0, ctypes.c_void_p(src.ctypes.data), nbytes, ctypes.byref(dev), _stream())
    expect = src.copy()
    src[:] = 0                                                      # the source may be reused as soon as the call returns
    L.call('hipcx_check_device_pointer', 0, dev)
    dev2 = ctypes.c_void_p()
    L.call('hipcx_malloc', 0, nbytes, ctypes.byref(dev2))
    L.call('hipcx_memcpy_device', 0, dev2, 0, dev, nbytes, _stream())
    back = np.empty(nbytes, np.uint8)
    L.call('hipcx_memcpy_to_host', 0, ctypes.c_void_p(back.ctypes.data), dev2, nbytes, _stream())
    assert np.array_equal(back, expect)
    # upload into existing memory (MemoryCopyFrom with a native source)
    reversed_bytes = back[::-1].copy()
    L.call('hipcx_memcpy_from_host', 0, dev, ctypes.c_void_p(reversed_bytes.ctypes.data), nbytes, _stream())
    again = np.empty(nbytes, np.uint8)
    L.call('hipcx_memcpy_to_host', 0, ctypes.c_void_p(again.ctypes.data), dev, nbytes, _stream())
    assert np.array_equal(again, expect[::-1])
    L.call('hipcx_free', 0, dev)
    L.call('hipcx_free', 0, dev2)


def test_foreign_pointer_check_rejects_host_memory():
    L = _lib()
    import chainer_amd as chx
    host = np.zeros(64, np.uint8)
    with pytest.raises(chx.ChainerxError):
        L.call('hipcx_check_device_pointer', 0, ctypes.c_void_p(host.ctypes.data))


def test_arrays_live_in_the_pool():
    import chainer_amd as chx
    chx.synchronize()
    base = chx.pool_stats()['in_use_blocks']
    a = chx.zeros((1000,), 'float32')
    b = a + a
    assert chx.pool_stats()['in_use_blocks'] == base + 2
    v = b[10:20]                                                    # a view keeps its buffer alive
    del b
    assert chx.pool_stats()['in_use_blocks'] == base + 2
    del v, a
    assert chx.pool_stats()['in_use_blocks'] == base


def test_graph_capture_in_an_arena_survives_other_allocations():
    """Replays of a captured graph stay correct while the general pool is churned: the graph's blocks belong to its arena."""
    import torch
    import chainer_amd as chx
    from chainer_amd.graph import capture
    rng = np.random.default_rng(5)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    w = rng.standard_normal((256, 256)).astype(np.float32) / 16
    X, W = chx.array(x), chx.array(w)

    def fn():
        h = chx.dot(X, W)
        h = chx.maximum(h, 0)
        return chx.sum(h * h, axis=1)

    eager = fn().get()
    g = capture(fn)
    for i in range(4):
        # eager work of the same sizes between the replays: it must not land on the graph's intermediates
        junk = [chx.zeros((64, 256), 'float32') + float(i) for _ in range(6)]
        g.replay()
        torch.cuda.synchronize()
        assert np.array_equal(g.result.get(), eager), 'replay %d' % i
        del junk
    g.release()


def test_record_stream_holds_a_freed_block_back():
    """A block allocated for one stream and used on another: after hipcx_record_stream its free waits for that stream, so the next
    allocation of its size class gets other memory while the foreign stream is busy and the block itself once it has caught up.
    Recording the block's own stream changes nothing."""
    import torch
    L = _lib()
    import chainer_amd as chx
    chx.synchronize()
    nbytes = 3 << 20
    p = ctypes.c_void_p()
    L.call('hipcx_malloc', 0, nbytes, ctypes.byref(p))  # the null stream's partition
    first = p.value
    L.call('hipcx_record_stream', 0, ctypes.c_void_p(first), ctypes.c_void_p(None))  # its own stream: immediate reuse
    L.call('hipcx_free', 0, ctypes.c_void_p(first))
    L.call('hipcx_malloc', 0, nbytes, ctypes.byref(p))
    assert p.value == first
    side = torch.cuda.Stream()
    a = torch.randn(8192, 8192, device='cuda')
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(24):  # a few hundred milliseconds of work queued on the side stream
            a = torch.mm(a, a) * 1e-4
    L.call('hipcx_record_stream', 0, ctypes.c_void_p(first), ctypes.c_void_p(side.cuda_stream))
    L.call('hipcx_free', 0, ctypes.c_void_p(first))
    busy = not side.query()
    L.call('hipcx_malloc', 0, nbytes, ctypes.byref(p))
    second = p.value
    if busy:
        assert second != first, 'the block was handed out again while the side stream could still use it'
    side.synchronize()
    L.call('hipcx_free', 0, ctypes.c_void_p(second))
    got = []
    for _ in range(2):  # both blocks of the class are free now
        L.call('hipcx_malloc', 0, nbytes, ctypes.byref(p))
        got.append(p.value)
    assert first in got
    for g in got:
        L.call('hipcx_free', 0, ctypes.c_void_p(g))
    with pytest.raises(chx.ChainerxError, match='not a block in use'):
        L.call('hipcx_record_stream', 0, ctypes.c_void_p(first), ctypes.c_void_p(side.cuda_stream))
    assert busy, 'the side stream finished before the free: the test did not exercise the hold-back'


def test_take_default_mode_is_captured_and_still_raises():
    """Take in the default bounds mode (mode=None, what the reference's callers pass) neither waits for the device nor reads a flag
    back, so a captured graph can hold it; an id that is out of range at replay time raises IndexError when the result is read."""
    import torch
    import chainer_amd as chx
    from chainer_amd.graph import capture
    rng = np.random.default_rng(9)
    table = rng.standard_normal((100, 64)).astype(np.float32)
    ids = rng.integers(0, 100, (32,)).astype(np.int32)
    T, I = chx.array(table), chx.array(ids)
    g = capture(lambda: chx.take(T, I, 0) * 2.0)
    g.replay()
    torch.cuda.synchronize()
    assert np.array_equal(g.result.get(), table[ids] * 2.0)
    I[5:6].fill(100)  # one past the end, written on the device
    g.replay()
    with pytest.raises(IndexError, match='Index 100 is out of bounds for axis 0 with size 100'):
        g.result.get()
    I[5:6].fill(-100)  # the lowest valid index
    g.replay()
    ids[5] = 0
    assert np.array_equal(g.result.get(), table[ids] * 2.0)
    g.release()


def test_graph_capture_refuses_a_function_that_keeps_allocating():
    """capture() warms a function up until one pass takes all its memory from the arena's free lists.  A function that keeps its
    results alive allocates new blocks in every pass: capture raises a clear error instead of calling the driver's allocator under
    stream capture."""
    import chainer_amd as chx
    from chainer_amd import graph
    hoard = []

    def grows():
        hoard.append(chx.zeros((256, 1024), 'float32') + 1.0)
        return hoard[-1]

    with pytest.raises(RuntimeError, match='warm passes'):
        graph.capture(grows)
    assert len(hoard) == graph.MAX_WARM_PASSES
    del hoard[:]
    # a function that settles after its first pass is captured as before
    x = chx.ones((64, 64), 'float32')
    g = graph.capture(lambda: x + x)
    g.replay()
    chx.synchronize()
    assert np.array_equal(g.result.get(), np.full((64, 64), 2, np.float32))
    g.release()

"""Kernels called from several host threads at once, each on a stream of its own, behind a barrier -- the pattern of the
reference's TEST_THREAD_SAFE_P (CX/testing/threading.h:34-60: every thread runs the same check concurrently).  ctypes releases
the interpreter lock for the duration of a call, so the library's host code really runs in parallel."""
import threading

import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact

pytestmark = pytest.mark.gpu

N_THREADS = 4
REPEATS = 6


def _worker(tid, barrier, failures):
    import torch
    import chainer_amd as chx
    try:
        rng = np.random.default_rng(100 + tid)
        stream = torch.cuda.Stream()
        # operands differ per thread, in sizes that exercise different kernels (and dynamic-LDS settings) at the same time
        n = 2 + tid
        x = rng.standard_normal((n, 32, 14, 14)).astype(np.float16)
        w3 = (rng.standard_normal((64, 32, 3, 3)) / 17).astype(np.float16)
        w1 = (rng.standard_normal((128, 32, 1, 1)) / 6).astype(np.float16)
        a = rng.standard_normal((96 + 8 * tid, 200)).astype(np.float32)
        b = (rng.standard_normal((200, 130)) / 14).astype(np.float32)
        r = rng.standard_normal((37 + tid, 5000)).astype(np.float32)
        ref_c3 = O.conv(x, w3, None, 1, 1, False)
        ref_c1 = O.conv(x, w1, None, 1, 0, False)
        ref_dot = O.dot(a, b)
        ref_sum = O.sum(r, axis=1)
        ref_arg = O.argmax(r, axis=1)
        ref_add = r + r
        with torch.cuda.stream(stream):
            X, W3, W1, A, B, R = (chx.array(v) for v in (x, w3, w1, a, b, r))
            barrier.wait()
            for _ in range(REPEATS):
                c3 = chx.conv(X, W3, None, 1, 1)
                c1 = chx.conv(X, W1, None, 1, 0)
                d = chx.dot(A, B)
                s = chx.sum(R, axis=1)
                am = chx.argmax(R, axis=1)
                e = R + R
                assert_close(c3.get(), ref_c3, 2e-2, 'thread %d conv3x3' % tid)
                assert_close(c1.get(), ref_c1, 2e-2, 'thread %d conv1x1' % tid)
                assert_close(d.get(), ref_dot, 1e-5, 'thread %d dot' % tid)
                assert_exact(s.get(), ref_sum, 'thread %d sum' % tid)
                assert_exact(am.get(), ref_arg, 'thread %d argmax' % tid)
                assert_exact(e.get(), ref_add, 'thread %d add' % tid)
        stream.synchronize()
    except BaseException as exc:  # reported by the main thread
        failures.append((tid, repr(exc)))
        try:
            barrier.abort()
        except Exception:
            pass


def test_concurrent_host_threads_on_their_own_streams():
    import chainer_amd as chx
    chx.synchronize()
    barrier = threading.Barrier(N_THREADS)
    failures = []
    threads = [threading.Thread(target=_worker, args=(t, barrier, failures)) for t in range(N_THREADS)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), 'a worker thread did not finish'
    assert not failures, failures
    chx.synchronize()

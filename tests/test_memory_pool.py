"""The backend's memory pool (chainer_amd/csrc/memory_pool.h) against a failing fake allocator, on the CPU: size classes, block
reuse, the release-and-retry path before OutOfMemoryError (CX/cuda/memory_pool.cc:236-243), deleters that outlive the pool
(CX/cuda/cuda_device/memory.cc:19-24), graph arenas, and four threads allocating at once.  The C++ test program is built with
g++ and run twice: plainly, and under ThreadSanitizer."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, 'tests', 'cpp', 'pool_test.cc')
INC = os.path.join(ROOT, 'chainer_amd', 'csrc')


def _build_and_run(tmp_path, extra_flags, name):
    exe = str(tmp_path / name)
    cmd = ['g++', '-std=c++17', '-O1', '-g', '-pthread', '-I', INC] + extra_flags + [SRC, '-o', exe]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return subprocess.run([exe], capture_output=True, text=True, timeout=300)


@pytest.mark.skipif(shutil.which('g++') is None, reason='g++ not available')
def test_memory_pool_behaviour(tmp_path):
    r = _build_and_run(tmp_path, [], 'pool_test')
    assert r.returncode == 0, r.stdout + r.stderr
    assert 'all checks passed' in r.stdout


@pytest.mark.skipif(shutil.which('g++') is None, reason='g++ not available')
def test_memory_pool_under_thread_sanitizer(tmp_path):
    try:
        r = _build_and_run(tmp_path, ['-fsanitize=thread'], 'pool_test_tsan')
    except subprocess.CalledProcessError as e:  # the sanitizer runtime is not installed everywhere
        pytest.skip('ThreadSanitizer build failed: %s' % e.stderr[-300:])
    if 'FATAL: ThreadSanitizer' in r.stderr and 'unexpected memory mapping' in r.stderr:
        pytest.skip('ThreadSanitizer cannot run in this address-space layout')
    assert r.returncode == 0 and 'WARNING: ThreadSanitizer' not in r.stderr, r.stdout + r.stderr[-3000:]

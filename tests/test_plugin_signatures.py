"""The ChainerX plugin glue (chainer_amd/plugin/hip_backend.cc) checked against the reference's own headers.

Needs the reference checkout (skipped without it; the GPU box has none) and hipcc.  Three checks:
  * the compiler's front end accepts the glue against chainerx/*.h: every `Call(...) override`, every
    `KernelRegistrar<HipBackend, Key, Impl>` and every Backend / Device member matches the signature it has to match
    (chainerx/kernel_registry.h:90-102, chainerx/backend.h, chainerx/device.h, chainerx/kernels/*.h);
  * compiled and linked as a shared object (ChainerX's own symbols left undefined, nothing is loaded or run), it exports the
    unmangled CreateBackend / DestroyBackend pair the loader looks up (chainerx/context.cc:84-111,
    chainerx/backend_testdata/backend0.cc:25-29);
  * every key kernel class declared in chainerx/kernels/*.h has a registration in the glue, except the ones listed by name.
abseil and gsl-lite, which ChainerX's headers include, are not in this image: tests/cpp/shim/ maps the handful of names used to
the standard library for this front-end check only (see its README).
"""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = '/root/reference/chainerx_cc'
GLUE = os.path.join(ROOT, 'chainer_amd', 'plugin', 'hip_backend.cc')
FLAGS = ['-std=c++17', '--offload-host-only', '-x', 'hip', '-Wno-unused-command-line-argument',
         '-I' + os.path.join(ROOT, 'tests', 'cpp', 'shim'), '-I' + REF, '-I' + os.path.join(ROOT, 'include')]

needs_reference = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, 'chainerx', 'kernels')) or shutil.which('hipcc') is None,
                                     reason='needs the reference checkout and hipcc')

# Key kernels without a registration, each with the reason: none.  (RnnKernel / RnnBackwardKernel are registered although the
# reference only dispatches them when the backend's name is "cuda", chainerx/routines/n_step_rnn.cc:210, :330; every other backend
# runs the routine's composition of registered kernels.)
NOT_REGISTERED = {}


@needs_reference
def test_glue_compiles_against_the_reference_headers():
    r = subprocess.run(['hipcc', '-fsyntax-only'] + FLAGS + [GLUE], capture_output=True, text=True, cwd=tempfile.gettempdir())
    assert r.returncode == 0, r.stderr[-4000:]


@needs_reference
def test_glue_exports_the_loader_entry_points():
    with tempfile.TemporaryDirectory() as tmp:
        obj = os.path.join(tmp, 'hip_backend.o')
        so = os.path.join(tmp, 'hip.so')
        r = subprocess.run(['hipcc', '-O0', '-fPIC', '-c'] + FLAGS + [GLUE, '-o', obj], capture_output=True, text=True, cwd=tmp)
        assert r.returncode == 0, r.stderr[-4000:]
        # symbols of libchainerx and of libhipcx stay undefined: this object is inspected, never loaded
        r = subprocess.run(['g++', '-shared', '-o', so, obj], capture_output=True, text=True, cwd=tmp)
        assert r.returncode == 0, r.stderr[-4000:]
        syms = subprocess.run(['nm', '-D', '--defined-only', so], capture_output=True, text=True).stdout
        defined = {line.split()[-1] for line in syms.splitlines() if line.strip()}
        assert 'CreateBackend' in defined and 'DestroyBackend' in defined, sorted(s for s in defined if 'Backend' in s)[:20]
        undefined = subprocess.run(['nm', '-D', '--undefined-only', so], capture_output=True, text=True).stdout
        used = set(re.findall(r'\b(hipcx_[a-z0-9_]+)\b', undefined))
        header = open(os.path.join(ROOT, 'include', 'hipcx.h')).read()
        declared = set(re.findall(r'\b(hipcx_[a-z0-9_]+)\s*\(', header))
        assert used and not (used - declared), sorted(used - declared)


@needs_reference
def test_every_key_kernel_is_registered():
    keys = set()
    kdir = os.path.join(REF, 'chainerx', 'kernels')
    for name in sorted(os.listdir(kdir)):
        if name.endswith('.h'):
            keys |= set(re.findall(r'class\s+(\w+Kernel)\s*:\s*public\s+Kernel\b', open(os.path.join(kdir, name)).read()))
    assert len(keys) > 100, len(keys)
    src = re.sub(r'//[^\n]*', '', open(GLUE).read())
    # direct registrations, and the macros that paste Name##Kernel
    registered = set(re.findall(r'HIPCX_REGISTER_KERNEL\(\s*(\w+Kernel)\s*,', src))
    macros = set(re.findall(r'#define\s+(HIPCX_\w+_KERNEL)\(Name', src))
    for macro in macros:
        registered |= {m + 'Kernel' for m in re.findall(r'^\s*' + macro + r'\(\s*(\w+)\s*,', src, re.M)}
    missing = keys - registered - set(NOT_REGISTERED)
    assert not missing, 'key kernels without a registration: %r' % sorted(missing)
    stale = set(NOT_REGISTERED) & registered
    assert not stale, 'listed as unregistered but registered: %r' % sorted(stale)
    unknown = registered - keys
    assert not unknown, 'registrations for classes the reference does not declare: %r' % sorted(unknown)

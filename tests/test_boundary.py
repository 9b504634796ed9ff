"""CPU tests of the drop-in boundary and the host-side routine layer (no kernel is launched here).

* the C-ABI library loads without a GPU and exports exactly the symbols include/hipcx.h declares, and the ctypes
  prototypes cover the same set;
* struct layouts seen from Python match the header;
* entry points that need no device (hipcx_conv_out_dim, argument validation) behave like the reference;
* dtype promotion, views, reshape and broadcasting follow ChainerX's rules (compared with numpy, which the reference's
  own Python tests use as the expected value).
"""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'hipcx.h')


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(hipcx_[a-z0-9_]+)\s*\(', text)))


def test_library_exports_every_declared_symbol():
    from chainer_amd import _lib
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 40
    out = subprocess.run(['nm', '-D', '--defined-only', _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = set(line.split()[-1] for line in out.splitlines() if ' T ' in line)
    for n in names:
        assert n in exported, '%s is declared in hipcx.h but not exported by libhipcx.so' % n
        getattr(lib, n)
    assert sorted(_lib.SIGNATURES) == names, 'ctypes prototypes and header disagree'
    # nothing undeclared leaks out under the hipcx_ prefix
    assert sorted(s for s in exported if s.startswith('hipcx_')) == names


def test_plugin_glue_only_forwards_to_declared_entry_points():
    """Checks of the plugin source that need no ChainerX checkout (test_plugin_signatures.py compiles it against one): every
    hipcx_* name it uses is declared in the header, and it reaches device memory only through those entry points."""
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = open(os.path.join(root, 'chainer_amd', 'plugin', 'hip_backend.cc')).read()
    header = open(os.path.join(root, 'include', 'hipcx.h')).read()
    declared = set(re.findall(r'\b(hipcx_[a-z0-9_]+)\s*\(', header))
    code = re.sub(r'//[^\n]*', '', src)
    used = set(re.findall(r'\b(hipcx_[a-z0-9_]+)\s*\(', code))
    assert used, 'no entry point found in the plugin source'
    assert not (used - declared), 'the plugin calls undeclared entry points: %r' % sorted(used - declared)
    for name in ('hipcx_malloc', 'hipcx_free', 'hipcx_from_host_memory', 'hipcx_memcpy_to_host', 'hipcx_memcpy_from_host',
                 'hipcx_memcpy_device', 'hipcx_check_device_pointer', 'hipcx_im2col', 'hipcx_col2im', 'hipcx_conv_transpose',
                 'hipcx_batch_norm_supported'):
        assert name in used, name
    for forbidden in ('hipMalloc', 'hipFree', 'hipMemcpy', 'hipMemset', 'hipLaunchKernelGGL', '__global__'):
        assert forbidden not in code, 'the plugin glue must not call %s itself' % forbidden


def test_struct_layouts_match_header():
    from chainer_amd import _lib
    assert ctypes.sizeof(_lib.CArray) == 8 + 4 + 4 + 8 * 10 + 8 * 10
    assert _lib.CArray.shape.offset == 16 and _lib.CArray.strides.offset == 96
    assert ctypes.sizeof(_lib.CScalar) == 24 and _lib.CScalar.i.offset == 8 and _lib.CScalar.f.offset == 16
    from chainer_amd import _array
    # chainerx::Dtype values (CX/dtype.h:19-29)
    assert [_array.dtype_code(d) for d in ('bool', 'int8', 'int16', 'int32', 'int64', 'uint8', 'float16', 'float32', 'float64')] == list(range(1, 10))


def test_version_and_error_reporting_without_device():
    from chainer_amd import _lib
    lib = _lib.load()
    assert lib.hipcx_version() >= 1
    # argument validation happens before any device work: a null array is an error with a message, not a crash
    st = lib.hipcx_exp(None, None, None)
    assert st != 0
    assert len(lib.hipcx_last_error()) > 0
    with pytest.raises(_lib.ChainerxError):
        _lib.check(st)


def test_conv_out_dim_entry_point():
    """GetConvOutDim (CX/routines/connection.cc:37-49) through the C ABI, against the definition."""
    from chainer_amd import _lib
    lib = _lib.load()
    for d in range(1, 30):
        for k in range(1, 6):
            for s in range(1, 4):
                for p in range(0, 3):
                    for cover in (0, 1):
                        num = d + 2 * p - k + (s - 1 if cover else 0)
                        exp = -1 if num < 0 else num // s + 1
                        assert lib.hipcx_conv_out_dim(d, k, s, p, cover) == exp
    assert lib.hipcx_conv_out_dim(224, 7, 2, 3, 0) == 112
    assert lib.hipcx_conv_out_dim(112, 3, 2, 0, 1) == 56 and lib.hipcx_conv_out_dim(112, 3, 2, 0, 0) == 55


def test_oracle_library_loads():
    from oracle import native
    L = native.lib()
    for name in ('oracle_float_to_half', 'oracle_half_to_float', 'oracle_sum_f32', 'oracle_argmax', 'oracle_dot_f32', 'oracle_conv_f16'):
        getattr(L, name)


def test_product_package_does_not_import_the_oracle():
    """The shipped path must not route through the CPU oracle."""
    pkg = os.path.join(ROOT, 'chainer_amd')
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(('.py', '.hip', '.h', '.cc')):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r'^\s*(from|import)\s+oracle\b', text, flags=re.M), '%s imports the oracle' % f
                assert 'liboracle' not in text and 'oracle/' not in text, '%s refers to the oracle library' % f


# ---------------------------------------------------------------------------------------------
# host logic: views over a host buffer (no kernels)
# ---------------------------------------------------------------------------------------------
def host_array(a):
    """chainer_amd.ndarray over host memory: enough for view arithmetic, never handed to a kernel."""
    import torch
    from chainer_amd._array import ndarray, contiguous_strides
    a = np.ascontiguousarray(a)
    buf = torch.from_numpy(a.reshape(-1).view(np.uint8).copy())
    return ndarray(buf, 0, a.shape, contiguous_strides(a.shape, a.dtype.itemsize), a.dtype)


def view_values(v):
    """Reads a view's elements back from its host buffer."""
    raw = v._buf.numpy()
    if v.size == 0:
        return np.empty(v.shape, v.dtype)
    lo = sum((d - 1) * s for d, s in zip(v.shape, v.strides) if s < 0)
    base = v._offset + lo
    return np.ndarray(v.shape, v.dtype, buffer=raw.tobytes()[base:], offset=-lo, strides=v.strides).copy()


def test_views_match_numpy():
    rng = np.random.default_rng(0)
    x = rng.integers(0, 1000, (4, 5, 6)).astype(np.int32)
    X = host_array(x)
    keys = [np.s_[1], np.s_[:, 2], np.s_[..., 3], np.s_[1:4:2, ::-1, 2:], np.s_[None, 2, :, None, 1], np.s_[-1, -2, -3], np.s_[::2, 1:1]]
    for key in keys:
        v = X[key]
        assert v.shape == x[key].shape, key
        assert np.array_equal(view_values(v), x[key]), key
    assert np.array_equal(view_values(X.transpose(2, 0, 1)), x.transpose(2, 0, 1))
    assert np.array_equal(view_values(X.T), x.T)
    assert np.array_equal(view_values(X[1].broadcast_to((3, 5, 6))), np.broadcast_to(x[1], (3, 5, 6)))
    assert X[:, :1].broadcast_to((4, 5, 6)).strides == (120, 0, 4)
    with pytest.raises(IndexError):
        X[4]
    from chainer_amd import DimensionError
    with pytest.raises(DimensionError):
        X.broadcast_to((4, 5, 7))
    with pytest.raises(DimensionError):
        X.transpose(0, 0, 1)


def test_reshape_is_a_view_exactly_when_strides_allow():
    """CX/routines/manipulation.cc:153-258: the same no-copy rule numpy uses."""
    x = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    X = host_array(x)
    for src, shape in [(np.s_[:], (6, 20)), (np.s_[:], (2, 3, 20)), (np.s_[:, :, :, :], (120,)), (np.s_[:, 1], (2, 20)),
                       (np.s_[:, :, ::2], (2, 3, 2, 5)), (np.s_[:, :, ::2], (6, 2, 5)), (np.s_[:, :, :, 0], (6, 4)), (np.s_[0], (1, 3, 1, 20))]:
        v = X[src]
        r = v.reshape(shape)  # only view-able cases listed: no kernel runs
        assert r._buf is X._buf
        assert np.array_equal(view_values(r), x[src].reshape(shape))
    # a transposed array cannot be flattened without a copy
    from chainer_amd._array import _nocopy_reshape_strides
    assert _nocopy_reshape_strides((3, 4), (4, 12), (12,), 4) is None
    assert _nocopy_reshape_strides((2, 3, 4), (48, 16, 4), (6, 4), 4) == (16, 4)
    assert _nocopy_reshape_strides((2, 3, 4), (96, 16, 4), (6, 4), 4) is None
    assert X.reshape(2, -1).shape == (2, 60)
    from chainer_amd import DimensionError
    with pytest.raises(DimensionError):
        X.reshape(7, -1)


def test_is_contiguous_ignores_unit_axes():
    """CX/shape.cc:15-32."""
    X = host_array(np.zeros((3, 1, 4), np.float32))
    assert X.is_contiguous and X[:, :, :].is_contiguous and X.transpose(1, 0, 2).is_contiguous
    assert not X.transpose(2, 1, 0).is_contiguous and not X[:, :, ::2].is_contiguous
    assert X[:1].transpose(2, 1, 0).shape == (4, 1, 1)


def test_dtype_promotion_table():
    """PromoteTypes / ResultType (CX/dtype.cc:12-60, CX/routines/type_util.cc:11-46): same as numpy for the nine dtypes,
    except that Python scalars never widen an array of the same or a higher category."""
    from chainer_amd import routines as R
    names = ['bool', 'int8', 'int16', 'int32', 'int64', 'uint8', 'float16', 'float32', 'float64']
    for a in names:
        for b in names:
            exp = np.promote_types(a, b)
            if {a, b} == {'uint8', 'int8'}:
                exp = np.dtype('int16')
            if np.dtype(a).kind in 'iu' and np.dtype(b).kind == 'f' or np.dtype(b).kind in 'iu' and np.dtype(a).kind == 'f':
                exp = np.dtype(a) if np.dtype(a).kind == 'f' else np.dtype(b)  # ints never widen a float (unlike numpy)
            if {np.dtype(a).kind, np.dtype(b).kind} == {'i', 'u'} and 'int8' not in (a, b):
                exp = np.dtype(a) if np.dtype(a).kind == 'i' else np.dtype(b)
            assert R.promote_types(a, b) == exp, (a, b)
    X16 = host_array(np.zeros(3, np.float16))
    Xi8 = host_array(np.zeros(3, np.int8))
    assert R.result_type(X16, 2.5) == np.float16 and R.result_type(X16, 3) == np.float16
    assert R.result_type(Xi8, 3) == np.int8 and R.result_type(Xi8, 2.5) == np.float32
    assert R.result_type(Xi8, X16) == np.float16


def test_scalar_kinds():
    """chainerx::Scalar keeps bool / int64 / double apart (CX/scalar.h)."""
    from chainer_amd import _lib
    assert _lib.make_scalar(True).kind == _lib.KIND_BOOL and _lib.make_scalar(True).i == 1
    assert _lib.make_scalar(-3).kind == _lib.KIND_INT and _lib.make_scalar(-3).i == -3
    assert _lib.make_scalar(np.float32(0.5)).kind == _lib.KIND_FLOAT and _lib.make_scalar(0.5).f == 0.5
    with pytest.raises(TypeError):
        _lib.make_scalar('x')


def test_no_device_means_loud_failure():
    import torch
    if torch.cuda.is_available():
        pytest.skip('a device is visible')
    import chainer_amd as chx
    with pytest.raises(chx.BackendError):
        chx.array(np.zeros(3, np.float32))
    with pytest.raises(chx.BackendError):
        chx.zeros((3,), 'float32')


def test_bench_rejects_more_than_one_gpu():
    r = subprocess.run(['python', os.path.join(ROOT, 'bench.py'), '--gpus', '2'], capture_output=True, text=True)
    assert r.returncode != 0 and 'one GPU' in (r.stderr + r.stdout)

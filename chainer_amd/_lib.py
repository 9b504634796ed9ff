"""ctypes binding of ``libhipcx.so`` (the C ABI declared in ``include/hipcx.h``).

The library is the only compute path of this package: if it is missing, or a call fails, an
exception is raised -- there is no CPU or PyTorch fallback.
"""
import ctypes
import os

MAX_NDIM = 10

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'libhipcx.so')


class ChainerxError(RuntimeError):
    """Base of the exceptions below; mirrors chainerx::ChainerxError (CX/error.h:48)."""


class DimensionError(ChainerxError):
    pass


class DtypeError(ChainerxError):
    pass


class ChainerxNotImplementedError(ChainerxError, NotImplementedError):
    pass


class ChainerxIndexError(ChainerxError, IndexError):
    pass


class BackendError(ChainerxError):
    pass


class DeviceError(ChainerxError):
    pass


class OutOfMemoryError(ChainerxError, MemoryError):
    """chainerx::cuda::OutOfMemoryError (CX/cuda/memory_pool.h:34-37)."""


_STATUS_TO_EXC = {
    1: ChainerxError,
    2: DimensionError,
    3: DtypeError,
    4: ChainerxNotImplementedError,
    5: ChainerxIndexError,
    6: BackendError,
    7: DeviceError,
    8: OutOfMemoryError,
}


class CArray(ctypes.Structure):
    _fields_ = [
        ('data', ctypes.c_void_p),
        ('dtype', ctypes.c_int32),
        ('ndim', ctypes.c_int32),
        ('shape', ctypes.c_int64 * MAX_NDIM),
        ('strides', ctypes.c_int64 * MAX_NDIM),
    ]


class CPoolStats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint64) for n in ('in_use_bytes', 'cached_bytes', 'in_use_blocks', 'cached_blocks',
                                               'device_allocations', 'retries')]


class CScalar(ctypes.Structure):
    _fields_ = [
        ('kind', ctypes.c_int32),
        ('reserved', ctypes.c_int32),
        ('i', ctypes.c_int64),
        ('f', ctypes.c_double),
    ]


KIND_BOOL, KIND_INT, KIND_FLOAT = 0, 1, 3


def make_scalar(value):
    """Python scalar -> hipcx_scalar with chainerx::Scalar's kind rule (CX/scalar.h)."""
    import numpy
    s = CScalar()
    if isinstance(value, (bool, numpy.bool_)):
        s.kind, s.i, s.f = KIND_BOOL, int(bool(value)), float(value)
    elif isinstance(value, (int, numpy.integer)):
        s.kind, s.i, s.f = KIND_INT, int(value), float(value)
    elif isinstance(value, (float, numpy.floating)):
        s.kind, s.i, s.f = KIND_FLOAT, 0, float(value)
    else:
        raise TypeError('unsupported scalar type: %r' % type(value))
    return s


_A = ctypes.POINTER(CArray)
_S = CScalar
_V = ctypes.c_void_p
_I8P = ctypes.POINTER(ctypes.c_int8)
_I64P = ctypes.POINTER(ctypes.c_int64)
_SZ = ctypes.c_size_t
_INT = ctypes.c_int

# name -> (restype, argtypes).  Every symbol declared in include/hipcx.h is listed here; the
# loader test checks the two against each other.
SIGNATURES = {
    'hipcx_last_error': (ctypes.c_char_p, []),
    'hipcx_version': (_INT, []),
    'hipcx_device_count': (_INT, [ctypes.POINTER(ctypes.c_int)]),
    'hipcx_synchronize': (_INT, [_INT]),
    'hipcx_record_stream': (_INT, [_INT, _V, _V]),
    'hipcx_device_name': (_INT, [_INT, ctypes.c_char_p, _SZ]),
    'hipcx_malloc': (_INT, [_INT, _SZ, ctypes.POINTER(ctypes.c_void_p)]),
    'hipcx_malloc_on_stream': (_INT, [_INT, _SZ, _V, ctypes.POINTER(ctypes.c_void_p)]),
    'hipcx_free': (_INT, [_INT, _V]),
    'hipcx_pool_free_unused': (_INT, [_INT]),
    'hipcx_pool_stats': (_INT, [_INT, ctypes.POINTER(CPoolStats)]),
    'hipcx_pool_set_arena': (_INT, [_INT, _INT]),
    'hipcx_pool_release_arena': (_INT, [_INT, _INT]),
    'hipcx_pool_destroy': (_INT, [_INT]),
    'hipcx_memcpy_from_host': (_INT, [_INT, _V, _V, _SZ, _V]),
    'hipcx_memcpy_to_host': (_INT, [_INT, _V, _V, _SZ, _V]),
    'hipcx_memcpy_device': (_INT, [_INT, _V, _INT, _V, _SZ, _V]),
    'hipcx_from_host_memory': (_INT, [_INT, _V, _SZ, ctypes.POINTER(ctypes.c_void_p), _V]),
    'hipcx_check_device_pointer': (_INT, [_INT, _V]),
    'hipcx_add': (_INT, [_A, _A, _A, _V]),
    'hipcx_add_as': (_INT, [_A, _S, _A, _V]),
    'hipcx_subtract': (_INT, [_A, _A, _A, _V]),
    'hipcx_subtract_as': (_INT, [_A, _S, _A, _V]),
    'hipcx_multiply': (_INT, [_A, _A, _A, _V]),
    'hipcx_multiply_as': (_INT, [_A, _S, _A, _V]),
    'hipcx_divide': (_INT, [_A, _A, _A, _V]),
    'hipcx_divide_as': (_INT, [_A, _S, _A, _V]),
    'hipcx_divide_sa': (_INT, [_S, _A, _A, _V]),
    'hipcx_exp': (_INT, [_A, _A, _V]),
    'hipcx_log': (_INT, [_A, _A, _V]),
    'hipcx_tanh': (_INT, [_A, _A, _V]),
    'hipcx_sqrt': (_INT, [_A, _A, _V]),
    'hipcx_if_less_else_assa': (_INT, [_A, _S, _S, _A, _A, _V]),
    'hipcx_if_greater_else_assa': (_INT, [_A, _S, _S, _A, _A, _V]),
    'hipcx_if_greater_else_aaaa': (_INT, [_A, _A, _A, _A, _A, _V]),
    'hipcx_equal': (_INT, [_A, _A, _A, _V]),
    'hipcx_not_equal': (_INT, [_A, _A, _A, _V]),
    'hipcx_greater': (_INT, [_A, _A, _A, _V]),
    'hipcx_greater_equal': (_INT, [_A, _A, _A, _V]),
    'hipcx_copy': (_INT, [_A, _A, _V]),
    'hipcx_fill': (_INT, [_A, _S, _V]),
    'hipcx_arange': (_INT, [_S, _S, _A, _V]),
    'hipcx_reduce_workspace_size': (_SZ, [_A, _I8P, _INT, _A]),
    'hipcx_sum': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_sum_static_scratch': (_INT, [_A, _I8P, _INT, _A, _V]),
    'hipcx_amax': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_argmax': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_dot_workspace_size': (_SZ, [_A, _A, _A]),
    'hipcx_dot': (_INT, [_A, _A, _A, _V, _SZ, _V]),
    'hipcx_conv_out_dim': (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, _INT]),
    'hipcx_conv_workspace_size': (_SZ, [_A, _A, _A]),
    'hipcx_conv': (_INT, [_A, _A, _A, _I64P, _I64P, _INT, _A, _V, _SZ, _V]),
    'hipcx_conv_route': (_INT, [_A, _A, _A, _I64P, _I64P, _A]),
    'hipcx_conv_bn_act': (_INT, [_A, _A, _A, _I64P, _I64P, _INT, _A, _A, _A, _A, _S, _A, _INT, _A, _V, _SZ, _V]),
    'hipcx_amin': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_argmin': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_all': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_any': (_INT, [_A, _I8P, _INT, _A, _V, _SZ, _V]),
    'hipcx_unary': (_INT, [_INT, _A, _A, _V]),
    'hipcx_predicate': (_INT, [_INT, _A, _A, _V]),
    'hipcx_logical': (_INT, [_INT, _A, _A, _A, _V]),
    'hipcx_power': (_INT, [_A, _A, _A, _V]),
    'hipcx_power_as': (_INT, [_A, _S, _A, _V]),
    'hipcx_power_sa': (_INT, [_S, _A, _A, _V]),
    'hipcx_binary': (_INT, [_INT, _A, _A, _A, _V]),
    'hipcx_binary_as': (_INT, [_INT, _A, _S, _A, _V]),
    'hipcx_binary_sa': (_INT, [_INT, _S, _A, _A, _V]),
    'hipcx_fmod': (_INT, [_A, _A, _A, _V]),
    'hipcx_arctan2': (_INT, [_A, _A, _A, _V]),
    'hipcx_where': (_INT, [_A, _A, _A, _A, _V]),
    'hipcx_where_aas': (_INT, [_A, _A, _S, _A, _V]),
    'hipcx_where_asa': (_INT, [_A, _S, _A, _A, _V]),
    'hipcx_where_ass': (_INT, [_A, _S, _S, _A, _V]),
    'hipcx_add_at': (_INT, [_A, _A, ctypes.c_int8, _A, _A, _INT, ctypes.POINTER(ctypes.c_int32), _V]),
    'hipcx_identity': (_INT, [_A, _V]),
    'hipcx_eye': (_INT, [ctypes.c_int64, _A, _V]),
    'hipcx_tri': (_INT, [ctypes.c_int64, _A, _V]),
    'hipcx_linspace': (_INT, [ctypes.c_double, ctypes.c_double, _A, _V]),
    'hipcx_diagflat': (_INT, [_A, ctypes.c_int64, _A, _V]),
    'hipcx_cumsum': (_INT, [_A, ctypes.c_int8, _A, _V]),
    'hipcx_log_softmax_workspace_size': (_SZ, [_A]),
    'hipcx_log_softmax': (_INT, [_A, _A, _V, _SZ, _V]),
    'hipcx_lstm_cell': (_INT, [_A, _A, _A, _A, _V]),
    'hipcx_profile_start': (_INT, []),
    'hipcx_profile_stop': (_INT, [_I64P, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double),
                                  ctypes.POINTER(ctypes.c_double)]),
    'hipcx_im2col': (_INT, [_A, _I64P, _I64P, _INT, _S, _A, _V]),
    'hipcx_col2im': (_INT, [_A, _I64P, _I64P, _A, _V]),
    'hipcx_conv_transpose_workspace_size': (_SZ, [_A, _A, _I64P, _I64P, _A]),
    'hipcx_conv_transpose': (_INT, [_A, _A, _A, _I64P, _I64P, _A, _V, _SZ, _V]),
    'hipcx_batch_norm_supported': (_INT, [_A, _I8P, _INT, ctypes.POINTER(_A), _INT]),
    'hipcx_n_step_lstm_workspace_size': (_SZ, [_INT, _A, ctypes.POINTER(_A), _INT]),
    'hipcx_n_step_lstm': (_INT, [_INT, _A, _A, ctypes.POINTER(_A), ctypes.POINTER(_A), ctypes.POINTER(_A), _INT, _A, _A, ctypes.POINTER(_A),
                                 _V, _SZ, _V]),
    'hipcx_n_step_rnn_reserve_size': (_SZ, [_INT, _INT, _INT, _A, ctypes.POINTER(_A), _INT]),
    'hipcx_n_step_rnn_workspace_size': (_SZ, [_INT, _INT, _INT, _INT, _A, ctypes.POINTER(_A), _INT]),
    'hipcx_n_step_rnn': (_INT, [_INT, _INT, _INT, _INT, _A, _A, ctypes.POINTER(_A), ctypes.POINTER(_A), ctypes.POINTER(_A), _INT, _A, _A,
                                ctypes.POINTER(_A), _V, _SZ, _V, _SZ, _V]),
    'hipcx_n_step_rnn_backward': (_INT, [_INT, _INT, _INT, _INT, _A, ctypes.POINTER(_A), ctypes.POINTER(_A), ctypes.POINTER(_A), _INT, _A, _A,
                                         ctypes.POINTER(_A), _V, _SZ, _A, _A, ctypes.POINTER(_A), ctypes.POINTER(_A), ctypes.POINTER(_A),
                                         _V, _SZ, _V]),
    'hipcx_profile_records': (_INT, [ctypes.c_int64, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double),
                                     ctypes.POINTER(ctypes.c_double), _I64P]),
    'hipcx_fixed_batch_norm': (_INT, [_A, _A, _A, _A, _A, _S, _I8P, _INT, _A, _V]),
    'hipcx_batch_norm_workspace_size': (_SZ, [_A, _I8P, _INT]),
    'hipcx_batch_norm': (_INT, [_A, _A, _A, _A, _A, _S, _S, _I8P, _INT, _A, _A, _A, _V, _SZ, _V]),
    'hipcx_batch_norm_grad': (_INT, [_A, _A, _A, _A, _A, _I8P, _INT, _A, _A, _A, _V, _SZ, _V]),
    'hipcx_solve_workspace_size': (_SZ, [_A]),
    'hipcx_solve': (_INT, [_A, _A, _A, _V, _SZ, ctypes.POINTER(ctypes.c_int32), _V]),
    'hipcx_inverse': (_INT, [_A, _A, _V, _SZ, ctypes.POINTER(ctypes.c_int32), _V]),
    'hipcx_cholesky': (_INT, [_A, _A, ctypes.POINTER(ctypes.c_int32), _V]),
    'hipcx_syevd_workspace_size': (_SZ, [_A]),
    'hipcx_syevd': (_INT, [_A, _A, _A, ctypes.c_char, _INT, _V, _SZ, _V]),
    'hipcx_qr_workspace_size': (_SZ, [_A]),
    'hipcx_qr': (_INT, [_A, _A, _A, _A, _INT, _V, _SZ, _V]),
    'hipcx_svd_workspace_size': (_SZ, [_A]),
    'hipcx_svd': (_INT, [_A, _A, _A, _A, _INT, _INT, _V, _SZ, _V]),
    'hipcx_conv_grad_weight_workspace_size': (_SZ, [_A, _A, _A, _I64P, _I64P, _INT]),
    'hipcx_conv_grad_weight': (_INT, [_A, _A, _I64P, _I64P, _INT, _A, _V, _SZ, _V]),
    'hipcx_max_pool': (_INT, [_A, _I64P, _I64P, _I64P, _INT, _A, _V]),
    'hipcx_average_pool': (_INT, [_A, _I64P, _I64P, _I64P, _INT, _A, _V]),
    'hipcx_max_pool_grad_workspace_size': (_SZ, [_A]),
    'hipcx_max_pool_grad': (_INT, [_A, _A, _I64P, _I64P, _I64P, _INT, _A, _V, _SZ, _V]),
    'hipcx_average_pool_grad': (_INT, [_A, _I64P, _I64P, _I64P, _INT, _A, _V]),
    'hipcx_max_pool_grad_grad': (_INT, [_A, _A, _I64P, _I64P, _I64P, _INT, _A, _V]),
    'hipcx_take': (_INT, [_A, _A, ctypes.c_int8, _A, _INT, ctypes.POINTER(ctypes.c_int32), _V]),
}

_lib = None


def load():
    """Loads libhipcx.so (once) and declares the prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            'libhipcx.so not found at %s: build it with `make -C chainer_amd/csrc` '
            '(or __graft_entry__.build()); there is no fallback path.' % LIB_PATH)
    # PyTorch owns the device buffers and the stream handed to every call, so the kernels must run
    # on the HIP runtime instance PyTorch has loaded: import it first, and the dynamic loader
    # resolves this library's libamdhip64 dependency to that already-loaded copy.
    import torch  # noqa: F401
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status):
    if status != 0:
        msg = load().hipcx_last_error().decode('utf-8', 'replace')
        raise _STATUS_TO_EXC.get(status, ChainerxError)(msg)


def call(name, *args):
    check(getattr(load(), name)(*args))

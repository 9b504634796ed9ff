"""Routines: the device-agnostic layer of ChainerX restated over the C ABI.

Each function mirrors one routine of ``CX/routines/*.cc``: the same dtype promotion, broadcasting,
output allocation and -- most importantly -- the same decomposition into kernel calls, one
``hipcx_*`` call per ``CallKernel<...>`` of the reference.  Nothing is fused here that the
reference does not fuse; the fused entry points live in ``chainer_amd.fused`` and are opt-in.
"""
import builtins as _py
import ctypes

import numpy

from chainer_amd import _lib
from chainer_amd._array import (ndarray, array, current_stream, alloc_bytes, _normalize_axis, _as_shape, _prod,
                                contiguous_strides)

# ---------------------------------------------------------------------------------------------
# dtype rules (CX/dtype.cc:12-60, CX/routines/type_util.cc:11-46)
# ---------------------------------------------------------------------------------------------
_KIND = {'b': 0, 'i': 1, 'u': 2, 'f': 3}
_CATEGORY = {0: 0, 1: 1, 2: 1, 3: 2}  # bool < int/uint < float


def _kind(dtype):
    return _KIND[numpy.dtype(dtype).kind]


def promote_types(dt1, dt2):
    dt1, dt2 = numpy.dtype(dt1), numpy.dtype(dt2)
    k1, k2 = _kind(dt1), _kind(dt2)
    if k1 == 0:
        return dt2
    if k2 == 0:
        return dt1
    if k1 == k2:
        return dt1 if dt1.itemsize >= dt2.itemsize else dt2
    if k1 == 3:
        return dt1
    if k2 == 3:
        return dt2
    if k1 == 2:
        dt1, dt2 = dt2, dt1
    if dt1.itemsize > dt2.itemsize:
        return dt1
    return numpy.dtype('int16')  # signed one level wider than uint8


def _scalar_default_dtype(value):
    if isinstance(value, (bool, numpy.bool_)):
        return numpy.dtype('bool')
    if isinstance(value, (int, numpy.integer)):
        return numpy.dtype('int32')
    return numpy.dtype('float32')


def result_type(*args):
    """ResultType over arrays and Python scalars: scalars only matter if of a higher category."""
    arr_dt = None
    sc_dt = None
    for a in args:
        if isinstance(a, ndarray):
            arr_dt = a.dtype if arr_dt is None else promote_types(arr_dt, a.dtype)
        else:
            d = _scalar_default_dtype(a)
            sc_dt = d if sc_dt is None else promote_types(sc_dt, d)
    if arr_dt is not None:
        if sc_dt is not None and _CATEGORY[_kind(sc_dt)] > _CATEGORY[_kind(arr_dt)]:
            return sc_dt
        return arr_dt
    return sc_dt


def _math_result_dtype(dtype):
    return numpy.dtype(dtype) if _kind(dtype) == 3 else numpy.dtype('float32')


def _is_scalar(x):
    return isinstance(x, (bool, int, float, numpy.bool_, numpy.integer, numpy.floating))


# ---------------------------------------------------------------------------------------------
# creation
# ---------------------------------------------------------------------------------------------
def empty(shape, dtype='float32'):
    return ndarray.empty(shape, dtype)


def empty_like(a):
    return ndarray.empty(a.shape, a.dtype)


def full(shape, value, dtype=None):
    if dtype is None:
        dtype = _scalar_default_dtype(value)
    out = ndarray.empty(shape, dtype)
    out.fill(value)
    return out


def zeros(shape, dtype='float32'):
    return full(shape, 0, dtype)


def ones(shape, dtype='float32'):
    return full(shape, 1, dtype)


def zeros_like(a):
    return zeros(a.shape, a.dtype)


def arange(start, stop=None, step=1, dtype=None):
    """Arange (CX/routines/creation.cc): size = ceil((stop-start)/step), then ArangeKernel."""
    if stop is None:
        start, stop = 0, start
    if dtype is None:
        dtype = result_type(start, stop, step)
        if _kind(dtype) == 0:
            dtype = numpy.dtype('int32')
    if step == 0:
        raise _lib.ChainerxError('Cannot create an arange array with 0 step size.')
    size = _py.max(0, int(numpy.ceil((stop - start) / step)))
    out = ndarray.empty((size,), dtype)
    _lib.call('hipcx_arange', _lib.make_scalar(start), _lib.make_scalar(step), out.desc(), current_stream())
    return out


def identity(n, dtype='float32'):
    """Identity (CX/routines/creation.cc:178-189)."""
    if n < 0:
        raise _lib.DimensionError('Negative dimensions are not allowed')
    out = ndarray.empty((n, n), dtype)
    if n:
        _lib.call('hipcx_identity', out.desc(), current_stream())
    return out


def eye(n, m=None, k=0, dtype='float64'):
    """Eye (CX/routines/creation.cc:191-211)."""
    m = n if m is None else m
    if n < 0 or m < 0:
        raise _lib.DimensionError('Negative dimensions are not allowed')
    out = ndarray.empty((n, m), dtype)
    if n * m:
        _lib.call('hipcx_eye', int(k or 0), out.desc(), current_stream())
    return out


def tri(n, m=None, k=0, dtype='float32'):
    """Tri (CX/routines/creation.cc:410-432)."""
    m = n if m is None else m
    if n < 0 or m < 0:
        raise _lib.DimensionError('Negative dimensions are not allowed')
    out = ndarray.empty((n, m), dtype)
    if n * m:
        _lib.call('hipcx_tri', int(k or 0), out.desc(), current_stream())
    return out


def linspace(start, stop, num=50, endpoint=True, dtype='float32'):
    """Linspace (CX/routines/creation.cc:313-339)."""
    if num < 0:
        raise _lib.ChainerxError('Number of samples, %d, must be non-negative' % num)
    out = ndarray.empty((num,), dtype)
    if num > 0:
        a, b = float(start), float(stop)
        if not endpoint:
            b = a + (b - a) * (num - 1) / num
        _lib.call('hipcx_linspace', a, b, out.desc(), current_stream())
    return out


def diag(v, k=0):
    """Diag (CX/routines/creation.cc:260-293): a 1-D v becomes the k-th diagonal of a square matrix; a 2-D v gives a view
    of its k-th diagonal."""
    if v.ndim == 1:
        n = v.shape[0] + abs(k)
        out = ndarray.empty((n, n), v.dtype)
        if n:
            _lib.call('hipcx_diagflat', v.desc(), int(k), out.desc(), current_stream())
        return out
    if v.ndim == 2:
        rows, cols = v.shape
        n = _py.min(rows, cols)
        if k >= 0:
            offset = k * v.strides[1]
            if cols <= k + n - 1:
                n = _py.max(0, cols - k)
        else:
            offset = -k * v.strides[0]
            if rows <= -k + n - 1:
                n = _py.max(0, rows + k)
        return ndarray(v._buf, v._offset + offset, (n,), (v.strides[0] + v.strides[1],), v.dtype)
    raise _lib.DimensionError('Input must be 1D or 2D.')


def diagflat(v, k=0):
    """Diagflat (CX/routines/creation.cc:307-310)."""
    return diag(v.reshape((_prod(v.shape),)), k)


def copy(a):
    return a.copy()


def ascontiguousarray(a):
    return a.as_contiguous()


def astype(a, dtype, copy=True):
    return a.astype(dtype, copy)


# ---------------------------------------------------------------------------------------------
# manipulation (views + Copy kernels)
# ---------------------------------------------------------------------------------------------
def reshape(a, shape):
    return a.reshape(shape)


def transpose(a, axes=None):
    return a.transpose(axes)


def broadcast_to(a, shape):
    return a.broadcast_to(shape)


def squeeze(a, axis=None):
    return a.squeeze(axis)


def split(a, indices_or_sections, axis=0):
    """Split into views (CX/routines/manipulation.cc Split)."""
    axis = _normalize_axis(axis, a.ndim)
    dim = a.shape[axis]
    if isinstance(indices_or_sections, (int, numpy.integer)):
        n = int(indices_or_sections)
        if n <= 0 or dim % n != 0:
            raise _lib.DimensionError('array split does not result in an equal division')
        step = dim // n
        bounds = [(i * step, (i + 1) * step) for i in range(n)]
    else:
        idx = [_py.min(_py.max(int(i), 0), dim) for i in indices_or_sections]
        starts = [0] + idx
        stops = idx + [dim]
        bounds = [(s, _py.max(s, e)) for s, e in zip(starts, stops)]
    out = []
    for s, e in bounds:
        key = [slice(None)] * a.ndim
        key[axis] = slice(s, e)
        out.append(a[tuple(key)])
    return out


def concatenate(arrays, axis=0):
    """Concatenate = Empty + one CopyKernel per input (CX/routines/manipulation.cc:415-460)."""
    arrays = list(arrays)
    if not arrays:
        raise _lib.DimensionError('Need at least one array to concatenate')
    axis = _normalize_axis(axis, arrays[0].ndim)
    dtype = arrays[0].dtype
    shape = list(arrays[0].shape)
    total = 0
    for a in arrays:
        if a.ndim != len(shape):
            raise _lib.DimensionError('all the input arrays must have same number of dimensions')
        for i in range(a.ndim):
            if i != axis and a.shape[i] != shape[i]:
                raise _lib.DimensionError('all the input array dimensions except for the concatenation axis must match exactly')
        total += a.shape[axis]
        dtype = promote_types(dtype, a.dtype)
    shape[axis] = total
    out = ndarray.empty(shape, dtype)
    pos = 0
    for a in arrays:
        key = [slice(None)] * out.ndim
        key[axis] = slice(pos, pos + a.shape[axis])
        _lib.call('hipcx_copy', a.desc(), out[tuple(key)].desc(), current_stream())
        pos += a.shape[axis]
    return out


# ---------------------------------------------------------------------------------------------
# elementwise
# ---------------------------------------------------------------------------------------------
def _broadcast_shape(s1, s2):
    n = _py.max(len(s1), len(s2))
    a = (1,) * (n - len(s1)) + tuple(s1)
    b = (1,) * (n - len(s2)) + tuple(s2)
    out = []
    for x, y in zip(a, b):
        if x == y or y == 1:
            out.append(x)
        elif x == 1:
            out.append(y)
        else:
            raise _lib.DimensionError('operands could not be broadcast together with shapes %r %r' % (tuple(s1), tuple(s2)))
    return tuple(out)


LAYOUT_FOLLOWS_INPUT = False


def _empty_for(x, shape, dtype):
    """Output allocation of the elementwise routines.  ChainerX routines call Empty(shape): C-contiguous.  With
    LAYOUT_FOLLOWS_INPUT (opt-in) a dense input's axis order is kept instead, so channels-last data stays channels-last."""
    if LAYOUT_FOLLOWS_INPUT and isinstance(x, ndarray) and x.shape == tuple(shape) and 0 not in x.strides:
        dtype = numpy.dtype(dtype)
        order = sorted(range(x.ndim), key=lambda i: (-abs(x.strides[i]), i))
        strides = [0] * x.ndim
        acc = dtype.itemsize
        for i in reversed(order):
            strides[i] = acc
            acc *= _py.max(1, x.shape[i])
        return ndarray(alloc_bytes(acc), 0, x.shape, strides, dtype)
    return ndarray.empty(shape, dtype)


def _binary(kernel, x1, x2, dtype, out=None):
    """BroadcastBinary (CX/routines/routines_util.h:53-72): operands arrive equal-shaped, cast to out's dtype."""
    shape = _broadcast_shape(x1.shape, x2.shape)
    a = x1 if x1.shape == shape else x1.broadcast_to(shape)
    b = x2 if x2.shape == shape else x2.broadcast_to(shape)
    if out is None:
        out = _empty_for(x1, shape, dtype)
    elif out.shape != shape:
        raise _lib.DimensionError('in-place operand shape %r does not match %r' % (out.shape, shape))
    _lib.call(kernel, a.astype(out.dtype, False).desc(), b.astype(out.dtype, False).desc(), out.desc(), current_stream())
    return out


def _binary_as(kernel, x1, scalar, dtype, out=None):
    if out is None:
        out = _empty_for(x1, x1.shape, dtype)
    _lib.call(kernel, x1.astype(out.dtype, False).desc(), _lib.make_scalar(scalar), out.desc(), current_stream())
    return out


def add(x1, x2, out=None):
    if _is_scalar(x2):
        return _binary_as('hipcx_add_as', x1, x2, result_type(x1, x2), out)
    if _is_scalar(x1):
        return _binary_as('hipcx_add_as', x2, x1, result_type(x1, x2), out)
    return _binary('hipcx_add', x1, x2, result_type(x1, x2), out)


def negative(x):
    """Negative = Multiply(x, Scalar{-1}) (CX/routines/arithmetic.cc)."""
    if x.dtype == numpy.dtype('bool'):
        raise _lib.DtypeError('Cannot negate a boolean array.')
    return _binary_as('hipcx_multiply_as', x, -1, x.dtype)


def subtract(x1, x2, out=None):
    dt = result_type(x1, x2)
    if _kind(dt) == 0:
        raise _lib.DtypeError('Boolean arguments are not supported in subtract.')
    if _is_scalar(x2):
        return _binary_as('hipcx_subtract_as', x1, x2, dt, out)
    if _is_scalar(x1):
        # Subtract(Scalar, Array) = Add(-Array, Scalar) (CX/routines/arithmetic.cc)
        return add(negative(x2), x1)
    return _binary('hipcx_subtract', x1, x2, dt, out)


def multiply(x1, x2, out=None):
    if _is_scalar(x2):
        return _binary_as('hipcx_multiply_as', x1, x2, result_type(x1, x2), out)
    if _is_scalar(x1):
        return _binary_as('hipcx_multiply_as', x2, x1, result_type(x1, x2), out)
    return _binary('hipcx_multiply', x1, x2, result_type(x1, x2), out)


def _true_divide_dtype(*args):
    dt = result_type(*args)
    return dt if _kind(dt) == 3 else numpy.dtype('float32')


def divide(x1, x2, out=None):
    """TrueDivide: integer operands are computed in float32 (CX/routines/arithmetic.cc Divide)."""
    dt = _true_divide_dtype(x1, x2)
    if _is_scalar(x2):
        return _binary_as('hipcx_divide_as', x1, x2, dt, out)
    if _is_scalar(x1):
        if out is None:
            out = ndarray.empty(x2.shape, dt)
        _lib.call('hipcx_divide_sa', _lib.make_scalar(x1), x2.astype(out.dtype, False).desc(), out.desc(), current_stream())
        return out
    return _binary('hipcx_divide', x1, x2, dt, out)


def reciprocal(x):
    """Reciprocal(x) = Scalar{1} / x (CX/routines/arithmetic.cc)."""
    return divide(1, x)


def _unary_math(kernel, x):
    dt = _math_result_dtype(x.dtype)
    xc = x.astype(dt, False)
    out = ndarray.empty(x.shape, dt)
    _lib.call(kernel, xc.desc(), out.desc(), current_stream())
    return out


def exp(x):
    return _unary_math('hipcx_exp', x)


def log(x):
    return _unary_math('hipcx_log', x)


def tanh(x):
    return _unary_math('hipcx_tanh', x)


def sqrt(x):
    return _unary_math('hipcx_sqrt', x)


def if_less_else(x1, x2, pos, neg):
    """x1 < x2 ? pos : neg with scalar x2/pos (CX/routines/misc.cc:34-58)."""
    dt = result_type(pos, neg)
    out = _empty_for(x1, x1.shape, dt)
    _lib.call('hipcx_if_less_else_assa', x1.astype(dt, False).desc(), _lib.make_scalar(x2), _lib.make_scalar(pos),
              neg.astype(dt, False).desc(), out.desc(), current_stream())
    return out


def if_greater_else(x1, x2, pos, neg):
    dt = result_type(pos, neg)
    out = ndarray.empty(x1.shape, dt)
    _lib.call('hipcx_if_greater_else_assa', x1.astype(dt, False).desc(), _lib.make_scalar(x2), _lib.make_scalar(pos),
              neg.astype(dt, False).desc(), out.desc(), current_stream())
    return out


def maximum(x1, x2):
    """Maximum(array, scalar) = IfLessElse(x1, x2, x2, x1) (CX/routines/misc.cc:210-216)."""
    if _is_scalar(x1):
        x1, x2 = x2, x1
    if _is_scalar(x2):
        return if_less_else(x1, x2, x2, x1)
    dt = result_type(x1, x2)
    shape = _broadcast_shape(x1.shape, x2.shape)
    a = x1.broadcast_to(shape).astype(dt, False)
    b = x2.broadcast_to(shape).astype(dt, False)
    out = ndarray.empty(shape, dt)
    # MaximumImpl: x1 > x2 ? x1 : x2 (CX/routines/misc.cc)
    _lib.call('hipcx_if_greater_else_aaaa', a.desc(), b.desc(), a.desc(), b.desc(), out.desc(), current_stream())
    return out


def minimum(x1, x2):
    if _is_scalar(x1):
        x1, x2 = x2, x1
    if _is_scalar(x2):
        return if_greater_else(x1, x2, x2, x1)
    raise _lib.ChainerxNotImplementedError('minimum(array, array) is not on the supported path')


def relu(x):
    """Relu(x) = Maximum(0, x) in the math dtype of x (CX/routines/activation.cc:80-84)."""
    return maximum(x.astype(_math_result_dtype(x.dtype), False), 0)


def sigmoid(x):
    """Sigmoid(x) = Reciprocal(1 + Exp(-x)): four kernels (CX/routines/activation.cc:74-78)."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    return reciprocal(add(exp(negative(xc)), 1))


def _compare(kernel, x1, x2):
    if _is_scalar(x2):
        x2 = full((), x2, x1.dtype)
    if (_kind(x1.dtype) == 0) != (_kind(x2.dtype) == 0):
        raise _lib.DtypeError('Comparison of bool and non-bool dtypes is not supported.')
    dt = promote_types(x1.dtype, x2.dtype)
    shape = _broadcast_shape(x1.shape, x2.shape)
    a = x1.broadcast_to(shape).astype(dt, False)
    b = x2.broadcast_to(shape).astype(dt, False)
    out = ndarray.empty(shape, 'bool')
    _lib.call(kernel, a.desc(), b.desc(), out.desc(), current_stream())
    return out


def equal(x1, x2):
    return _compare('hipcx_equal', x1, x2)


def not_equal(x1, x2):
    return _compare('hipcx_not_equal', x1, x2)


def greater(x1, x2):
    return _compare('hipcx_greater', x1, x2)


def greater_equal(x1, x2):
    return _compare('hipcx_greater_equal', x1, x2)


def less(x1, x2):
    """Less(x1, x2) = Greater(x2, x1) (CX/routines/logic.h:33)."""
    return greater(x2, x1)


def less_equal(x1, x2):
    """LessEqual(x1, x2) = GreaterEqual(x2, x1) (CX/routines/logic.h:38)."""
    return greater_equal(x2, x1)


# Op codes of include/hipcx.h (enum hipcx_unary_op / hipcx_predicate_op / hipcx_logical_op).
_UNARY_CODES = {name: i + 1 for i, name in enumerate(
    ['erf', 'expm1', 'exp2', 'log10', 'log2', 'log1p', 'sinh', 'cosh', 'arcsinh', 'arccosh', 'sin', 'cos', 'tan', 'arcsin',
     'arccos', 'arctan', 'ceil', 'floor', 'square', 'absolute', 'sign'])}
_PRED_CODES = {'logical_not': 1, 'isnan': 2, 'isinf': 3, 'isfinite': 4}
_LOGICAL_CODES = {'logical_and': 1, 'logical_or': 2, 'logical_xor': 3}


def _float_unary(name, x):
    """Unary math routines: the result dtype is x's float dtype, float32 for other kinds (GetMathResultDtype)."""
    dt = _math_result_dtype(x.dtype)
    out = ndarray.empty(x.shape, dt)
    _lib.call('hipcx_unary', _UNARY_CODES[name], x.astype(dt, False).desc(), out.desc(), current_stream())
    return out


def erf(x):
    return _float_unary('erf', x)


def expm1(x):
    return _float_unary('expm1', x)


def exp2(x):
    return _float_unary('exp2', x)


def log10(x):
    return _float_unary('log10', x)


def log2(x):
    return _float_unary('log2', x)


def log1p(x):
    return _float_unary('log1p', x)


def sinh(x):
    return _float_unary('sinh', x)


def cosh(x):
    return _float_unary('cosh', x)


def arcsinh(x):
    return _float_unary('arcsinh', x)


def arccosh(x):
    return _float_unary('arccosh', x)


def sin(x):
    return _float_unary('sin', x)


def cos(x):
    return _float_unary('cos', x)


def tan(x):
    return _float_unary('tan', x)


def arcsin(x):
    return _float_unary('arcsin', x)


def arccos(x):
    return _float_unary('arccos', x)


def arctan(x):
    return _float_unary('arctan', x)


def ceil(x):
    return _float_unary('ceil', x)


def floor(x):
    return _float_unary('floor', x)


def _numeric_unary(name, x, message):
    if x.dtype == numpy.dtype('bool'):
        raise _lib.DtypeError(message)
    out = ndarray.empty(x.shape, x.dtype)
    _lib.call('hipcx_unary', _UNARY_CODES[name], x.desc(), out.desc(), current_stream())
    return out


def square(x):
    """Square (CX/routines/misc.cc:141-150)."""
    return _numeric_unary('square', x, "Square operation don't support Boolean type")


def absolute(x):
    """Absolute (CX/routines/misc.cc:185-192)."""
    return _numeric_unary('absolute', x, 'Absolute does not support boolean array')


def fabs(x):
    """Fabs (CX/routines/misc.cc:194-199): Absolute into the math result dtype."""
    return absolute(x.astype(_math_result_dtype(x.dtype), False))


def sign(x):
    """Sign (CX/routines/misc.cc:201-208); the kernel visits numeric dtypes only."""
    return _numeric_unary('sign', x, 'bool dtype is not supported by this kernel')


def _predicate(name, x):
    out = ndarray.empty(x.shape, 'bool')
    _lib.call('hipcx_predicate', _PRED_CODES[name], x.desc(), out.desc(), current_stream())
    return out


def logical_not(x):
    return _predicate('logical_not', x)


def isnan(x):
    return _predicate('isnan', x)


def isinf(x):
    return _predicate('isinf', x)


def isfinite(x):
    return _predicate('isfinite', x)


def _logical(name, x1, x2):
    """LogicBinary (CX/routines/logic.cc:36-41): bool with non-bool is a DtypeError; the kernel promotes the operands."""
    if (_kind(x1.dtype) == 0) != (_kind(x2.dtype) == 0):
        raise _lib.DtypeError('Comparison of bool and non-bool dtypes is not supported.')
    dt = promote_types(x1.dtype, x2.dtype)
    shape = _broadcast_shape(x1.shape, x2.shape)
    a = x1.broadcast_to(shape).astype(dt, False)
    b = x2.broadcast_to(shape).astype(dt, False)
    out = ndarray.empty(shape, 'bool')
    _lib.call('hipcx_logical', _LOGICAL_CODES[name], a.desc(), b.desc(), out.desc(), current_stream())
    return out


def logical_and(x1, x2):
    return _logical('logical_and', x1, x2)


def logical_or(x1, x2):
    return _logical('logical_or', x1, x2)


def logical_xor(x1, x2):
    return _logical('logical_xor', x1, x2)


def _arithmetic_dtype(x1, x2):
    """GetArithmeticResultDtype (CX/routines/arithmetic.cc:28-61): bool operands are refused."""
    k1 = _kind(_scalar_default_dtype(x1)) if _is_scalar(x1) else _kind(x1.dtype)
    k2 = _kind(_scalar_default_dtype(x2)) if _is_scalar(x2) else _kind(x2.dtype)
    if k1 == 0 or k2 == 0:
        raise _lib.DtypeError('Boolean arguments are not allowed in arithmetic functions.')
    return result_type(x1, x2)


def power(x1, x2):
    """Power (CX/routines/arithmetic.cc:487-491)."""
    dt = _arithmetic_dtype(x1, x2)
    if _is_scalar(x2):
        return _binary_as('hipcx_power_as', x1, x2, dt)
    if _is_scalar(x1):
        out = ndarray.empty(x2.shape, dt)
        _lib.call('hipcx_power_sa', _lib.make_scalar(x1), x2.astype(dt, False).desc(), out.desc(), current_stream())
        return out
    return _binary('hipcx_power', x1, x2, dt)


def fmod(x1, x2):
    """Fmod (CX/routines/arithmetic.cc:607); the kernel visits float dtypes only."""
    dt = _arithmetic_dtype(x1, x2)
    if _kind(dt) != 3:
        raise _lib.DtypeError('floating point dtype required, got %s' % dt)
    return _binary('hipcx_fmod', x1, x2, dt)


def arctan2(x1, x2):
    """Arctan2 (CX/routines/trigonometric.cc:150-151): computed in the math result dtype of the operands."""
    return _binary('hipcx_arctan2', x1, x2, _math_result_dtype(result_type(x1, x2)))


_BINARY_CODES = {'floor_divide': 1, 'mod': 2, 'bitwise_and': 3, 'bitwise_or': 4, 'bitwise_xor': 5, 'left_shift': 6, 'right_shift': 7}


def _binary_code(name, x1, x2, dtype):
    """array op array (broadcast), array op scalar, scalar op array through hipcx_binary / _as / _sa."""
    code = _BINARY_CODES[name]
    if _is_scalar(x2):
        out = ndarray.empty(x1.shape, dtype)
        _lib.call('hipcx_binary_as', code, x1.astype(dtype, False).desc(), _lib.make_scalar(x2), out.desc(), current_stream())
        return out
    if _is_scalar(x1):
        out = ndarray.empty(x2.shape, dtype)
        _lib.call('hipcx_binary_sa', code, _lib.make_scalar(x1), x2.astype(dtype, False).desc(), out.desc(), current_stream())
        return out
    shape = _broadcast_shape(x1.shape, x2.shape)
    out = ndarray.empty(shape, dtype)
    _lib.call('hipcx_binary', code, x1.broadcast_to(shape).astype(dtype, False).desc(), x2.broadcast_to(shape).astype(dtype, False).desc(),
              out.desc(), current_stream())
    return out


def floor_divide(x1, x2):
    """FloorDivide (CX/routines/arithmetic.cc:305-311)."""
    return _binary_code('floor_divide', x1, x2, _arithmetic_dtype(x1, x2))


def mod(x1, x2):
    """Mod (CX/routines/arithmetic.cc:568-572)."""
    return _binary_code('mod', x1, x2, _arithmetic_dtype(x1, x2))


remainder = mod


def _operand_kind(x):
    return _kind(_scalar_default_dtype(x)) if _is_scalar(x) else _kind(x.dtype)


def _bitwise(name, x1, x2):
    """BitwiseAnd / Or / Xor (CX/routines/binary.cc:19-23,125-159): float operands are refused; Scalar op Array swaps."""
    if _operand_kind(x1) == 3 or _operand_kind(x2) == 3:
        raise _lib.DtypeError("Bitwise operations don't support Float types")
    if _is_scalar(x1):
        x1, x2 = x2, x1
    return _binary_code(name, x1, x2, result_type(x1, x2))


def bitwise_and(x1, x2):
    return _bitwise('bitwise_and', x1, x2)


def bitwise_or(x1, x2):
    return _bitwise('bitwise_or', x1, x2)


def bitwise_xor(x1, x2):
    return _bitwise('bitwise_xor', x1, x2)


def _shift(name, x1, x2):
    """LeftShift / RightShift (CX/routines/binary.cc:32-36,161-189): integer operands only; the result has x1's dtype,
    int64 when x1 is a scalar."""
    if _operand_kind(x1) in (0, 3) or _operand_kind(x2) in (0, 3):
        raise _lib.DtypeError("Shift operations don't support Float or Bool types")
    return _binary_code(name, x1, x2, numpy.dtype('int64') if _is_scalar(x1) else x1.dtype)


def left_shift(x1, x2):
    return _shift('left_shift', x1, x2)


def right_shift(x1, x2):
    return _shift('right_shift', x1, x2)


def where(condition, x, y):
    """Where (CX/routines/indexing.cc:207-298): out dtype = ResultType(x, y); a non-bool condition is cast to bool."""
    cond = condition.astype('bool', False)
    dt = result_type(x, y)
    xs, ys = _is_scalar(x), _is_scalar(y)
    shape = cond.shape
    if not xs:
        shape = _broadcast_shape(shape, x.shape)
    if not ys:
        shape = _broadcast_shape(shape, y.shape)
    out = ndarray.empty(shape, dt)
    c = cond.broadcast_to(shape)
    if xs and ys:
        _lib.call('hipcx_where_ass', c.desc(), _lib.make_scalar(x), _lib.make_scalar(y), out.desc(), current_stream())
    elif ys:
        _lib.call('hipcx_where_aas', c.desc(), x.broadcast_to(shape).astype(dt, False).desc(), _lib.make_scalar(y), out.desc(), current_stream())
    elif xs:
        _lib.call('hipcx_where_asa', c.desc(), _lib.make_scalar(x), y.broadcast_to(shape).astype(dt, False).desc(), out.desc(), current_stream())
    else:
        _lib.call('hipcx_where', c.desc(), x.broadcast_to(shape).astype(dt, False).desc(), y.broadcast_to(shape).astype(dt, False).desc(),
                  out.desc(), current_stream())
    return out


# ---------------------------------------------------------------------------------------------
# reductions
# ---------------------------------------------------------------------------------------------
def _sorted_axes(axis, ndim):
    if axis is None:
        return tuple(range(ndim))
    if isinstance(axis, (int, numpy.integer)):
        axis = (axis,)
    ax = sorted(_normalize_axis(a, ndim) for a in axis)
    if len(set(ax)) != len(ax):
        raise _lib.DimensionError('Duplicate axis values.')
    return tuple(ax)


def _reduced_out(a, axes, keepdims, dtype):
    """EmptyReduced (CX/routines/creation.cc:56-75): kept axes get stride 0."""
    if keepdims:
        out_shape = [1 if i in axes else d for i, d in enumerate(a.shape)]
        inner = [d for i, d in enumerate(a.shape) if i not in axes]
        inner_strides = list(contiguous_strides(inner, numpy.dtype(dtype).itemsize))
        strides = []
        for i in range(a.ndim):
            strides.append(0 if i in axes else inner_strides.pop(0))
        nbytes = _prod(inner) * numpy.dtype(dtype).itemsize
        return ndarray(alloc_bytes(nbytes), 0, out_shape, strides, dtype)
    return ndarray.empty([d for i, d in enumerate(a.shape) if i not in axes], dtype)


def _reduce(kernel, a, axes, out):
    n = len(axes)
    ax = (ctypes.c_int8 * _py.max(n, 1))(*axes)
    ws_bytes = _lib.load().hipcx_reduce_workspace_size(a.desc(), ax, n, out.desc())
    ws = alloc_bytes(ws_bytes) if ws_bytes else None
    _lib.call(kernel, a.desc(), ax, n, out.desc(), ctypes.c_void_p(ws.data_ptr() if ws is not None else 0), ws_bytes, current_stream())
    return out


def sum(a, axis=None, keepdims=False):
    """Sum (CX/routines/reduction.cc:28-76): bool/int inputs accumulate and return int64."""
    axes = _sorted_axes(axis, a.ndim)
    k = _kind(a.dtype)
    out_dtype = numpy.dtype('int64') if k in (0, 1, 2) else a.dtype
    out = _reduced_out(a, axes, keepdims, out_dtype)
    return _reduce('hipcx_sum', a, axes, out)


def amax(a, axis=None, keepdims=False):
    """AMax (CX/routines/statistics.cc:21-65)."""
    axes = _sorted_axes(axis, a.ndim)
    for i in axes:
        if a.shape[i] == 0:
            raise _lib.DimensionError('cannot compute the maximum along zero-sized axis')
    out = _reduced_out(a, axes, keepdims, a.dtype)
    return _reduce('hipcx_amax', a, axes, out)


max = amax


def argmax(a, axis=None):
    """ArgMax (CX/routines/sorting.cc:21-52): int64 result, no keepdims."""
    axes = _sorted_axes(axis, a.ndim)
    for i in axes:
        if a.shape[i] == 0:
            raise _lib.DimensionError('cannot compute ArgMax for an empty array')
    out = ndarray.empty([d for i, d in enumerate(a.shape) if i not in axes], 'int64')
    return _reduce('hipcx_argmax', a, axes, out)


def amin(a, axis=None, keepdims=False):
    """AMin (CX/routines/statistics.cc:66-79)."""
    axes = _sorted_axes(axis, a.ndim)
    for i in axes:
        if a.shape[i] == 0:
            raise _lib.DimensionError('cannot compute the minimum along zero-sized axis')
    out = _reduced_out(a, axes, keepdims, a.dtype)
    return _reduce('hipcx_amin', a, axes, out)


min = amin


def argmin(a, axis=None):
    """ArgMin (CX/routines/sorting.cc:54-85): int64 result, no keepdims."""
    axes = _sorted_axes(axis, a.ndim)
    for i in axes:
        if a.shape[i] == 0:
            raise _lib.DimensionError('cannot compute ArgMin for an empty array')
    out = ndarray.empty([d for i, d in enumerate(a.shape) if i not in axes], 'int64')
    return _reduce('hipcx_argmin', a, axes, out)


def nanargmax(a, axis=None):
    """NanArgMax (CX/routines/sorting.cc:93-126): NaNs replaced by -inf, then the ArgMax kernel (the native NanArgMaxKernel is
    its ArgMax functor, native/native_device/reduction.cc:171-198)."""
    return argmax(where(isnan(a), float('-inf'), a), axis)


def nanargmin(a, axis=None):
    """NanArgMin (CX/routines/sorting.cc): NaNs replaced by +inf, then the ArgMin kernel."""
    return argmin(where(isnan(a), float('inf'), a), axis)


def all(a, axis=None, keepdims=False):
    """All (CX/routines/logic.cc:79-87); the kernel casts the input to bool first (native/native_device/logic.cc)."""
    axes = _sorted_axes(axis, a.ndim)
    out = _reduced_out(a, axes, keepdims, 'bool')
    return _reduce('hipcx_all', a.astype('bool', False), axes, out)


def any(a, axis=None, keepdims=False):
    """Any (CX/routines/logic.cc:89-97)."""
    axes = _sorted_axes(axis, a.ndim)
    out = _reduced_out(a, axes, keepdims, 'bool')
    return _reduce('hipcx_any', a.astype('bool', False), axes, out)


def cumsum(a, axis=None):
    """Cumsum (CX/routines/reduction.cc:103-134): over the flattened array when axis is None; bool / integer inputs give int64."""
    if axis is None:
        a = a.reshape((_prod(a.shape),))
        axis = 0
    else:
        axis = _normalize_axis(axis, a.ndim)
    out = ndarray.empty(a.shape, 'int64' if _kind(a.dtype) in (0, 1, 2) else a.dtype)
    if _prod(a.shape):
        _lib.call('hipcx_cumsum', a.desc(), axis, out.desc(), current_stream())
    return out


def nansum(a, axis=None, keepdims=False):
    """Nansum (CX/routines/reduction.cc:149-170): Where(IsNan(a), 0, a), then the sum kernel (the native NansumKernel is its
    SumKernel, native/native_device/reduction.cc:146-167)."""
    return sum(where(isnan(a), 0, a), axis, keepdims)


def mean(a, axis=None, keepdims=False):
    """Mean = Sum then DivideAS by the item count (CX/routines/statistics.cc:95-154)."""
    axes = _sorted_axes(axis, a.ndim)
    dt = a.dtype if _kind(a.dtype) == 3 else numpy.dtype('float32')
    out = _reduced_out(a, axes, keepdims, dt)
    _reduce('hipcx_sum', a, axes, out)
    n = _prod([a.shape[i] for i in axes])
    _lib.call('hipcx_divide_as', out.desc(), _lib.make_scalar(int(n)), out.desc(), current_stream())
    return out


def logsumexp(x, axis=None, keepdims=False):
    """LogSumExp (CX/routines/reduction.cc:78-86): AMax, Subtract, Exp, Sum, Log, Add."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    axes = _sorted_axes(axis, x.ndim)
    xmax = amax(xc, axes, True)
    logs = log(sum(exp(subtract(xc, xmax)), axes, keepdims))
    return add(xmax if keepdims else xmax.squeeze(axes), logs)


def log_softmax(x, axis=None):
    """LogSoftmax = x - LogSumExp(x, axis or 1, keepdims) (CX/routines/reduction.cc:88-92): seven kernels."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    return subtract(xc, logsumexp(xc, 1 if axis is None else axis, True))


def log_softmax_fused(x, axis=None):
    """Opt-in: LogSoftmax (CX/routines/reduction.cc:88-92) through hipcx_log_softmax -- one or two kernels instead of seven.
    Arrays the fused kernel does not take (ndim != 2, another axis, strided rows) go through log_softmax."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    ax = 1 if axis is None else axis
    axes = _sorted_axes(ax, x.ndim)
    it = xc.dtype.itemsize
    if xc.ndim != 2 or axes != (1,) or (xc.shape[1] > 1 and xc.strides[1] != it) or xc.strides[0] < 0:
        return log_softmax(x, axis)
    out = ndarray.empty(xc.shape, xc.dtype)
    nbytes = _lib.load().hipcx_log_softmax_workspace_size(xc.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_log_softmax', xc.desc(), out.desc(), wsp, nbytes, current_stream())
    return out


def softmax(x, axis=None):
    """Softmax (CX/routines/reduction.cc:68-76)."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    axes = _sorted_axes(1 if axis is None else axis, x.ndim)
    xmax = amax(xc, axes, True)
    exps = exp(subtract(xc, xmax))
    sums = sum(exps, axes, True)
    return multiply(exps, reciprocal(sums))


# ---------------------------------------------------------------------------------------------
# linear algebra / connection
# ---------------------------------------------------------------------------------------------
def _workspace(nbytes):
    if not nbytes:
        return None, ctypes.c_void_p(0)
    ws = alloc_bytes(nbytes)
    return ws, ctypes.c_void_p(ws.data_ptr())


def dot(a, b, out_dtype=None):
    """Dot for 2-D operands (CX/routines/linalg.cc:27-100): k == 0 gives zeros without a kernel."""
    if a.ndim != 2 or b.ndim != 2:
        raise _lib.DimensionError('ChainerX dot supports only 2-dimensional arrays.')
    if a.shape[1] != b.shape[0]:
        raise _lib.DimensionError('Axis dimension mismatch')
    dt = numpy.dtype(out_dtype) if out_dtype is not None else result_type(a, b)
    m, k, n = a.shape[0], a.shape[1], b.shape[1]
    if k == 0:
        return zeros((m, n), dt)
    out = ndarray.empty((m, n), dt)
    _dot_into(a.astype(dt, False), b.astype(dt, False), out)
    return out


def _dot_into(a, b, out):
    nbytes = _lib.load().hipcx_dot_workspace_size(a.desc(), b.desc(), out.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_dot', a.desc(), b.desc(), out.desc(), wsp, nbytes, current_stream())


def linear(x, w, b=None, n_batch_axes=1):
    """Linear (CX/routines/connection.cc:322-394): DotKernel(x, w.T view) then AddKernel with a stride-0 bias."""
    if w.ndim != 2:
        raise _lib.DimensionError('w.ndim should be 2')
    if b is not None and b.ndim != 1:
        raise _lib.DimensionError('b.ndim should be 1')
    n_batch_axes = _normalize_axis(n_batch_axes, x.ndim) if x.ndim > 0 else 0
    dt = result_type(x, w, b) if b is not None else result_type(x, w)
    out_dim = _prod(x.shape[:n_batch_axes])
    m_dim, n_dim = w.shape
    out_shape = tuple(x.shape[:n_batch_axes]) + (m_dim,)
    if m_dim == 0 or n_dim == 0:
        if b is not None:
            return b.astype(dt, False).broadcast_to(out_shape)
        return zeros(out_shape, dt)
    x_matrix = x.reshape(out_dim, n_dim)
    out_matrix = ndarray.empty((out_dim, m_dim), dt)
    _dot_into(x_matrix.astype(dt, False), w.transpose().astype(dt, False), out_matrix)
    if b is not None:
        b_matrix = b.broadcast_to((out_dim, m_dim))
        _lib.call('hipcx_add', out_matrix.desc(), b_matrix.astype(dt, False).desc(), out_matrix.desc(), current_stream())
    return out_matrix.reshape(out_shape)


def _pair(v, n=2):
    if isinstance(v, (int, numpy.integer)):
        return (int(v),) * n
    v = tuple(int(i) for i in v)
    if len(v) != n:
        raise _lib.DimensionError('expected %d values, got %r' % (n, v))
    return v


def _i64(values):
    return (ctypes.c_int64 * len(values))(*values)


def conv_out_dim(in_dim, kernel_size, stride, pad, cover_all):
    n = _lib.load().hipcx_conv_out_dim(in_dim, kernel_size, stride, pad, int(bool(cover_all)))
    if n < 0:
        raise _lib.DimensionError('Output size should be positive.')
    return n


def _channels_last_empty(n, c, h, w, dtype):
    """NCHW-shaped array over NHWC memory (the layout the native backend's own conv result has)."""
    it = numpy.dtype(dtype).itemsize
    strides = (h * w * c * it, it, w * c * it, c * it)
    return ndarray(alloc_bytes(n * c * h * w * it), 0, (n, c, h, w), strides, dtype)


def _is_channels_last(x):
    return x.ndim == 4 and x.strides[1] == x.itemsize and x.shape[1] > 1 and (x.shape[2] * x.shape[3] > 1)


def _spatial_out(x, n, c, h, w, dtype):
    """Output of the kernels that allocate their own result (Conv, MaxPool, AveragePool).  C-contiguous NCHW, like the
    CUDA backend's (CX/cuda/cuda_conv.cc:311); channels-last when the opt-in LAYOUT_FOLLOWS_INPUT mode is on and the
    input already is."""
    if LAYOUT_FOLLOWS_INPUT and (_is_channels_last(x) or x.shape[1] < 8):
        return _channels_last_empty(n, c, h, w, dtype)
    return ndarray.empty((n, c, h, w), dtype)


def conv(x, w, b=None, stride=1, pad=0, cover_all=False, out_dtype=None):
    """Conv (CX/routines/connection.cc:140-208): one ConvKernel call with the bias inside.  Any number of spatial axes; the
    dedicated kernels are the 2-D ones (0 and 1 axes run through them as extents of one, 3 and more through a plain kernel)."""
    if x.ndim < 2 or w.ndim != x.ndim:
        raise _lib.DimensionError('Mismatched number of dimensions in input %r and weights %r.' % (x.shape, w.shape))
    n = x.ndim - 2
    stride, pad = _pair(stride, n), _pair(pad, n)
    if w.shape[1] != x.shape[1]:
        raise _lib.DimensionError('Mismatched number of input channels in input %r and weights %r.' % (x.shape, w.shape))
    if b is not None and (b.ndim != 1 or b.shape[0] != w.shape[0]):
        raise _lib.DimensionError('Mismatched bias shape %r for weights %r.' % (b.shape, w.shape))
    dt = numpy.dtype(out_dtype) if out_dtype is not None else (result_type(x, w, b) if b is not None else result_type(x, w))
    dims = tuple(conv_out_dim(x.shape[2 + d], w.shape[2 + d], stride[d], pad[d], cover_all) for d in range(n))
    out = _spatial_out(x, x.shape[0], w.shape[0], dims[0], dims[1], dt) if n == 2 else ndarray.empty((x.shape[0], w.shape[0]) + dims, dt)
    xc, wc = x.astype(dt, False), w.astype(dt, False)
    bc = b.astype(dt, False) if b is not None else None
    nbytes = _lib.load().hipcx_conv_workspace_size(xc.desc(), wc.desc(), out.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_conv', xc.desc(), wc.desc(), bc.desc() if bc is not None else None, _i64(stride), _i64(pad),
              int(bool(cover_all)), out.desc(), wsp, nbytes, current_stream())
    return out


def conv_route(x, w, b=None, stride=1, pad=0, cover_all=False):
    """Which kernel family `conv` runs for these arguments (hipcx_conv_route): 0 general implicit GEMM, 1 float16 NCHW kernels
    with 128-wide tiles, 2 the 7x7 / 2 stem kernel, 3 the float16 1x1 kernel with LDS-direct operand loads.  For tests and
    benchmarks; not part of the ChainerX routine surface."""
    stride, pad = _pair(stride), _pair(pad)
    dt = result_type(x, w, b) if b is not None else result_type(x, w)
    oh = conv_out_dim(x.shape[2], w.shape[2], stride[0], pad[0], cover_all)
    ow = conv_out_dim(x.shape[3], w.shape[3], stride[1], pad[1], cover_all)
    out = _spatial_out(x, x.shape[0], w.shape[0], oh, ow, dt)
    xc, wc = x.astype(dt, False), w.astype(dt, False)
    bc = b.astype(dt, False) if b is not None else None
    return int(_lib.load().hipcx_conv_route(xc.desc(), wc.desc(), bc.desc() if bc is not None else None, _i64(stride), _i64(pad), out.desc()))


def conv_bn_act(x, w, b=None, stride=1, pad=0, cover_all=False, bn=None, eps=2e-5, residual=None, relu=False):
    """Opt-in fused block: relu(fixed_batch_norm(conv(x, w, b), *bn, eps, axis=(0, 2, 3)) + residual) in one kernel call.
    `bn` is None or (gamma, beta, mean, var), one value per output channel.  Not part of the ChainerX routine surface:
    the reference issues these as separate kernels (which `conv`, `fixed_batch_norm`, `add`, `relu` here do as well)."""
    if x.ndim != 4 or w.ndim != 4:
        raise _lib.ChainerxNotImplementedError('only 2-D convolution is on the supported path')
    stride, pad = _pair(stride), _pair(pad)
    if w.shape[1] != x.shape[1]:
        raise _lib.DimensionError('Mismatched number of input channels in input %r and weights %r.' % (x.shape, w.shape))
    dt = result_type(x, w)
    oh = conv_out_dim(x.shape[2], w.shape[2], stride[0], pad[0], cover_all)
    ow = conv_out_dim(x.shape[3], w.shape[3], stride[1], pad[1], cover_all)
    out = _spatial_out(x, x.shape[0], w.shape[0], oh, ow, dt)
    xc, wc = x.astype(dt, False), w.astype(dt, False)
    bc = b.astype(dt, False) if b is not None else None
    prm = [a.astype(dt, False).desc() for a in bn] if bn is not None else [None] * 4
    res = residual.astype(dt, False) if residual is not None else None
    nbytes = _lib.load().hipcx_conv_workspace_size(xc.desc(), wc.desc(), out.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_conv_bn_act', xc.desc(), wc.desc(), bc.desc() if bc is not None else None, _i64(stride), _i64(pad),
              int(bool(cover_all)), prm[0], prm[1], prm[2], prm[3], _lib.make_scalar(float(eps)),
              res.desc() if res is not None else None, int(bool(relu)), out.desc(), wsp, nbytes, current_stream())
    return out


def fixed_batch_norm(x, gamma, beta, mean, var, eps=2e-5, axis=None):
    """FixedBatchNorm (CX/routines/normalization.cc:414-424 with PreprocessBatchNorm :61-101)."""
    for a in (x, gamma, beta, mean, var):
        if _kind(a.dtype) != 3:
            raise _lib.DtypeError('BatchNorm only supports floating kind inputs.')
    axes = _sorted_axes(axis, x.ndim) if axis is not None else (0,)
    reduced_shape = tuple(1 if i in axes else d for i, d in enumerate(x.shape))
    size = _prod(reduced_shape)
    params = []
    for name, a in (('Gamma', gamma), ('Beta', beta), ('Mean', mean), ('Variance', var)):
        if a.size != size:
            raise _lib.DimensionError('%s must have the same size as the reduced input. Actual: %d. Expected: %d.' % (name, a.size, size))
        params.append(a.reshape(reduced_shape))
    out = ndarray(alloc_bytes(x.nbytes), 0, x.shape, _dense_strides_like(x), x.dtype)
    ax = (ctypes.c_int8 * len(axes))(*axes)
    _lib.call('hipcx_fixed_batch_norm', x.desc(), params[0].desc(), params[1].desc(), params[2].desc(), params[3].desc(),
              _lib.make_scalar(float(eps)), ax, len(axes), out.desc(), current_stream())
    return out


def _dense_strides_like(x):
    """Dense strides with the same axis order as x's memory (so a channels-last input gives a channels-last output)."""
    order = sorted(range(x.ndim), key=lambda i: (-abs(x.strides[i]), i))
    strides = [0] * x.ndim
    acc = x.itemsize
    for i in reversed(order):
        strides[i] = acc
        acc *= _py.max(1, x.shape[i])
    return tuple(strides)


def max_pool(x, ksize, stride=None, pad=0, cover_all=False):
    """MaxPool (CX/routines/pooling.cc:52-123); one or more spatial axes (the dedicated kernels are the 2-D ones)."""
    if x.ndim < 3:
        raise _lib.DimensionError('pooling needs at least one spatial axis, got the shape %r' % (x.shape,))
    n = x.ndim - 2
    ksize = _pair(ksize, n)
    stride = ksize if stride is None else _pair(stride, n)
    pad = _pair(pad, n)
    dims = tuple(conv_out_dim(x.shape[2 + d], ksize[d], stride[d], pad[d], cover_all) for d in range(n))
    out = _spatial_out(x, x.shape[0], x.shape[1], dims[0], dims[1], x.dtype) if n == 2 else ndarray.empty(x.shape[:2] + dims, x.dtype)
    _lib.call('hipcx_max_pool', x.desc(), _i64(ksize), _i64(stride), _i64(pad), int(bool(cover_all)), out.desc(), current_stream())
    return out


def average_pool(x, ksize, stride=None, pad=0, pad_mode='ignore'):
    """AveragePool (CX/routines/pooling.cc:125-169), float dtypes only; one or more spatial axes."""
    if _kind(x.dtype) != 3:
        raise _lib.DtypeError('cannot apply average pooling to non-float arrays')
    if x.ndim < 3:
        raise _lib.DimensionError('pooling needs at least one spatial axis, got the shape %r' % (x.shape,))
    n = x.ndim - 2
    ksize = _pair(ksize, n)
    stride = ksize if stride is None else _pair(stride, n)
    pad = _pair(pad, n)
    mode = {'zero': 1, 'ignore': 2}[pad_mode]
    dims = tuple(conv_out_dim(x.shape[2 + d], ksize[d], stride[d], pad[d], False) for d in range(n))
    out = _spatial_out(x, x.shape[0], x.shape[1], dims[0], dims[1], x.dtype) if n == 2 else ndarray.empty(x.shape[:2] + dims, x.dtype)
    _lib.call('hipcx_average_pool', x.desc(), _i64(ksize), _i64(stride), _i64(pad), mode, out.desc(), current_stream())
    return out


# ---------------------------------------------------------------------------------------------
# linear algebra (CX/routines/linalg.cc): solve, inv, cholesky, eigh, eigvalsh, qr, svd, pinv
# ---------------------------------------------------------------------------------------------
def _check_square(a):
    if a.ndim != 2:
        raise _lib.DimensionError('ChainerX linear algebra routines only support 2-dimensional arrays.')
    if a.shape[0] != a.shape[1]:
        raise _lib.DimensionError('Matrix is not square.')


def _linalg_flag():
    flag = zeros((1,), 'int32')
    return flag, ctypes.cast(ctypes.c_void_p(flag.data_ptr), ctypes.POINTER(ctypes.c_int32))


def _raise_if_flagged(flag, what):
    info = int(flag.get()[0])
    if info != 0:
        raise _lib.ChainerxError('Unsuccessful %s execution. Info = %d' % (what, info))


def solve(a, b):
    """Solve (CX/routines/linalg.cc:121-163): x with a @ x = b, b a vector or a matrix; dtype = ResultType(a, b)."""
    _check_square(a)
    dt = result_type(a, b)
    if dt == numpy.dtype('float16'):
        raise _lib.DtypeError('Half-precision (float16) is not supported by solve')
    if _kind(dt) != 3:
        dt = numpy.dtype('float32') if dt.itemsize < 8 else numpy.dtype('float64')
    out = ndarray.empty(b.shape, dt)
    nbytes = _lib.load().hipcx_solve_workspace_size(a.desc())
    ws, wsp = _workspace(nbytes)
    flag, flag_ptr = _linalg_flag()
    _lib.call('hipcx_solve', a.desc(), b.desc(), out.desc(), wsp, nbytes, flag_ptr, current_stream())
    _raise_if_flagged(flag, 'gesv (Solve)')
    return out


def inv(a):
    """Inverse (CX/routines/linalg.cc:165-192), in the math dtype of a."""
    _check_square(a)
    dt = _math_result_dtype(a.dtype)
    if dt == numpy.dtype('float16'):
        raise _lib.DtypeError('Half-precision (float16) is not supported by inverse')
    out = ndarray.empty(a.shape, dt)
    nbytes = _lib.load().hipcx_solve_workspace_size(a.desc())
    ws, wsp = _workspace(nbytes)
    flag, flag_ptr = _linalg_flag()
    _lib.call('hipcx_inverse', a.desc(), out.desc(), wsp, nbytes, flag_ptr, current_stream())
    _raise_if_flagged(flag, 'getrf (LU)')
    return out


def cholesky(a):
    """Cholesky (CX/routines/linalg.cc:415-450): the lower factor L of a = L @ L.T, read from a's lower triangle."""
    _check_square(a)
    dt = _math_result_dtype(a.dtype)
    if dt == numpy.dtype('float16'):
        raise _lib.DtypeError('Half-precision (float16) is not supported by cholesky')
    out = ndarray.empty(a.shape, dt)
    flag, flag_ptr = _linalg_flag()
    _lib.call('hipcx_cholesky', a.desc(), out.desc(), flag_ptr, current_stream())
    _raise_if_flagged(flag, 'potrf (Cholesky)')
    return out


def _syevd(a, uplo, compute_v):
    _check_square(a)
    if not isinstance(uplo, str) or len(uplo) != 1:
        raise TypeError('UPLO must be a one-character string')
    if uplo.upper() not in ('U', 'L'):
        raise _lib.ChainerxError("UPLO argument must be 'L' or 'U'.")
    if a.dtype == numpy.dtype('float16'):
        raise _lib.DtypeError('Half-precision (float16) is not supported by eigen decomposition')
    if _kind(a.dtype) != 3:
        raise _lib.DtypeError('Eigen decomposition needs a floating-point matrix')
    w = ndarray.empty((a.shape[0],), a.dtype)
    v = ndarray.empty(a.shape, a.dtype)
    nbytes = _lib.load().hipcx_syevd_workspace_size(a.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_syevd', a.desc(), w.desc(), v.desc(), uplo.encode(), 1 if compute_v else 0, wsp, nbytes, current_stream())
    return w, v


def eigh(a, UPLO='L'):
    """Eigh (CX/routines/linalg.cc:452-495): (w, v) with a @ v = v * w, w ascending, a read from its UPLO triangle."""
    return _syevd(a, UPLO, True)


def eigvalsh(a, UPLO='L'):
    """Eigvalsh (CX/routines/linalg.cc:497-511): the eigenvalues alone."""
    return _syevd(a, UPLO, False)[0]


_QR_MODES = {'reduced': 0, 'complete': 1, 'r': 2, 'raw': 3}


def qr(a, mode='reduced'):
    """Qr (CX/routines/linalg.cc:333-413; mode strings CX/python/routines.cc:450-477): (q, r) for 'reduced' / 'complete', r for
    'r', (h, tau) for 'raw' (h = the factored matrix, transposed: LAPACK's column-major result)."""
    if a.ndim != 2:
        raise _lib.DimensionError('ChainerX linear algebra routines only support 2-dimensional arrays.')
    if mode not in _QR_MODES:
        raise ValueError("mode must be 'reduced', 'complete', 'r', or 'raw'")
    if a.dtype == numpy.dtype('float16'):
        raise _lib.DtypeError('Half-precision (float16) is not supported by QR decomposition')
    if _kind(a.dtype) != 3:
        raise _lib.DtypeError('QR decomposition needs a floating-point matrix')
    m, n = a.shape
    k = _py.min(m, n)
    dt = a.dtype
    tau = ndarray.empty((k,), dt)
    q = None
    if mode == 'reduced':
        q, r = ndarray.empty((m, k), dt), ndarray.empty((k, n), dt)
    elif mode == 'complete':
        q, r = ndarray.empty((m, m), dt), ndarray.empty((m, n), dt)
    elif mode == 'r':
        r = ndarray.empty((k, n), dt)
    else:
        r = ndarray.empty((n, m), dt)
    nbytes = _lib.load().hipcx_qr_workspace_size(a.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_qr', a.desc(), q.desc() if q is not None else None, r.desc(), tau.desc(), _QR_MODES[mode], wsp, nbytes,
              current_stream())
    if mode == 'r':
        return r
    if mode == 'raw':
        return r, tau
    return q, r


def svd(a, full_matrices=True, compute_uv=True):
    """Svd (CX/routines/linalg.cc:194-301; defaults CX/python/routines.cc:429-443): (u, s, vt) with a = u @ diag(s) @ vt, s
    descending; s alone without compute_uv."""
    if a.ndim != 2:
        raise _lib.DimensionError('ChainerX linear algebra routines only support 2-dimensional arrays.')
    if a.dtype == numpy.dtype('float16'):
        raise _lib.DtypeError('Half-precision (float16) is not supported by SVD')
    if _kind(a.dtype) != 3:
        raise _lib.DtypeError('SVD needs a floating-point matrix')
    m, n = a.shape
    k = _py.min(m, n)
    dt = a.dtype
    s = ndarray.empty((k,), dt)
    u = vt = None
    if compute_uv:
        u = ndarray.empty((m, m if full_matrices else k), dt)
        vt = ndarray.empty((n if full_matrices else k, n), dt)
    nbytes = _lib.load().hipcx_svd_workspace_size(a.desc())
    ws, wsp = _workspace(nbytes)
    _lib.call('hipcx_svd', a.desc(), u.desc() if compute_uv else None, s.desc(), vt.desc() if compute_uv else None,
              1 if full_matrices else 0, 1 if compute_uv else 0, wsp, nbytes, current_stream())
    return (u, s, vt) if compute_uv else s


def pinv(a, rcond=1e-15):
    """PseudoInverse (CX/routines/linalg.cc:303-331): vt.T @ diag(1 / s, 0 where s <= rcond * max(s)) @ u.T from the reduced SVD."""
    u, s, vt = svd(a, full_matrices=False, compute_uv=True)
    if a.size == 0:
        return copy(a.T)
    cutoff = multiply(amax(s), float(numpy.float32(rcond)))
    sinv = where(less_equal(s, cutoff), 0, reciprocal(s))
    return dot(multiply(vt.T, sinv), u.T)


# ---------------------------------------------------------------------------------------------
# indexing
# ---------------------------------------------------------------------------------------------
_BOUNDS = {None: 0, 'raise': 1, 'wrap': 2, 'clip': 3}


def take(a, indices, axis, mode=None):
    """Take (CX/routines/indexing.cc:171-205).  mode 'raise' raises IndexError on out-of-range ids from this call, like the native
    backend (one 4-byte read-back after the kernel).  mode None -- what the reference's callers pass -- raises it too, but late: the
    kernel records the bad index on the device and the next call that waits for the device (``get`` / ``synchronize``) raises, so
    a loop of take calls never waits for the host and can be captured into a graph."""
    if _kind(indices.dtype) not in (1, 2):
        raise _lib.DtypeError('Only arrays of integer dtype can be used as indices.')
    axis = _normalize_axis(axis, a.ndim)
    out_shape = a.shape[:axis] + indices.shape + a.shape[axis + 1:]
    out = ndarray.empty(out_shape, a.dtype)
    m = _BOUNDS[mode]
    flag = None
    flag_ptr = None
    if m == 1:
        flag = zeros((1,), 'int32')
        flag_ptr = ctypes.cast(ctypes.c_void_p(flag.data_ptr), ctypes.POINTER(ctypes.c_int32))
    _lib.call('hipcx_take', a.desc(), indices.desc(), axis, out.desc(), m, flag_ptr, current_stream())
    if flag is not None and int(flag.get()[0]) != 0:
        raise _lib.ChainerxIndexError('Index is out of bounds for axis %d with size %d' % (axis, a.shape[axis]))
    return out


def add_at(a, indices, axis, b, mode=None):
    """AddAt kernel call as Take's backward issues it (CX/routines/indexing.cc:147-169): a copy of a with b added at the
    indexed positions of `axis`; repeated indices accumulate in index order."""
    if _kind(indices.dtype) not in (1, 2):
        raise _lib.DtypeError('Only arrays of integer dtype can be used as indices.')
    axis = _normalize_axis(axis, a.ndim)
    if b.shape != a.shape[:axis] + indices.shape + a.shape[axis + 1:]:
        raise _lib.DimensionError('b has the wrong shape')
    out = ndarray.empty(a.shape, a.dtype)
    m = _BOUNDS[mode]
    flag = None
    flag_ptr = None
    if m == 1:
        flag = zeros((1,), 'int32')
        flag_ptr = ctypes.cast(ctypes.c_void_p(flag.data_ptr), ctypes.POINTER(ctypes.c_int32))
    _lib.call('hipcx_add_at', a.desc(), indices.desc(), axis, b.astype(a.dtype, False).desc(), out.desc(), m, flag_ptr, current_stream())
    if flag is not None and int(flag.get()[0]) != 0:
        raise _lib.ChainerxIndexError('Index is out of bounds for axis %d with size %d' % (axis, a.shape[axis]))
    return out


# ---------------------------------------------------------------------------------------------
# backward / training kernels, composed from the kernels above exactly as the reference's native backend composes them
# (Im2Col / Col2Im as strided Copy / Add kernel calls, TensorDot as transposes + Dot)
# ---------------------------------------------------------------------------------------------
def _copy_into(dst_view, src):
    _lib.call('hipcx_copy', src.desc(), dst_view.desc(), current_stream())


# True: Im2Col / Col2Im run as the native backend's chains of strided Copy / Add kernel calls instead of one launch each.
COMPOSE_IM2COL = False


def im2col(x, ksize, stride, pad, cover_all=False, pad_value=0):
    """native_internal::Im2Col (CX/native/im2col.cc:82-149): col[N, C, kh, kw, oh, ow] -- one hipcx_im2col launch, or (COMPOSE_IM2COL)
    a padded copy of x and one strided Copy per kernel offset as the native backend does it."""
    n, c, h, w = x.shape
    kh, kw = ksize
    sh, sw = stride
    ph, pw = pad
    oh = conv_out_dim(h, kh, sh, ph, cover_all)
    ow = conv_out_dim(w, kw, sw, pw, cover_all)
    if not COMPOSE_IM2COL:
        col = ndarray.empty((n, c, kh, kw, oh, ow), x.dtype)
        _lib.call('hipcx_im2col', x.desc(), _i64((sh, sw)), _i64((ph, pw)), int(bool(cover_all)), _lib.make_scalar(pad_value), col.desc(),
                  current_stream())
        return col
    hp = h + 2 * ph + (sh - 1 if cover_all else 0)
    wp = w + 2 * pw + (sw - 1 if cover_all else 0)
    xp = full((n, c, hp, wp), pad_value, x.dtype)
    _copy_into(xp[:, :, ph:ph + h, pw:pw + w], x)
    col = ndarray.empty((n, c, kh, kw, oh, ow), x.dtype)
    for r in range(kh):
        for q in range(kw):
            _copy_into(col[:, :, r, q], xp[:, :, r:r + sh * oh:sh, q:q + sw * ow:sw])
    return col


def col2im(col, stride, pad, out_size):
    """native_internal::Col2Im (CX/native/col2im.cc:76-122): zeros of the padded size, then for every kernel offset in (r, s)
    order an in-place strided Add -- the accumulation order of the reference -- and a view without the padding."""
    n, c, kh, kw, h, w = col.shape
    sh, sw = stride
    ph, pw = pad
    oh, ow = out_size
    if not COMPOSE_IM2COL:  # one launch: every image position sums its contributions in the same order, with the same roundings
        out = ndarray.empty((n, c, oh, ow), col.dtype)
        _lib.call('hipcx_col2im', col.desc(), _i64((sh, sw)), _i64((ph, pw)), out.desc(), current_stream())
        return out
    padded = zeros((n, c, oh + 2 * ph + sh - 1, ow + 2 * pw + sw - 1), col.dtype)
    for r in range(kh):
        for q in range(kw):
            view = padded[:, :, r:r + sh * h:sh, q:q + sw * w:sw]
            _lib.call('hipcx_add', view.desc(), col[:, :, r, q].desc(), view.desc(), current_stream())
    return padded[:, :, ph:ph + oh, pw:pw + ow]


def tensordot(a, b, a_axes, b_axes, out_dtype=None):
    """TensorDot (CX/native/tensor_dot.cc:63-99): reduced axes of a rolled last, of b rolled first, reshape to 2-D, Dot."""
    a_axes = [ax % a.ndim for ax in a_axes]
    b_axes = [ax % b.ndim for ax in b_axes]
    a_keep = [i for i in range(a.ndim) if i not in a_axes]
    b_keep = [i for i in range(b.ndim) if i not in b_axes]
    red = _prod([a.shape[i] for i in a_axes])
    a2 = a.transpose(a_keep + a_axes).reshape((_prod([a.shape[i] for i in a_keep]), red))
    b2 = b.transpose(b_axes + b_keep).reshape((red, _prod([b.shape[i] for i in b_keep])))
    out = dot(a2, b2, out_dtype)
    return out.reshape(tuple(a.shape[i] for i in a_keep) + tuple(b.shape[i] for i in b_keep))


# True: ConvGradWeight runs as strided copies + Dot issued from here instead of through hipcx_conv_grad_weight.
COMPOSE_CONV_GRAD_WEIGHT = False


def _conv_grad_weight_nd(w_dtype, w_shape, x, gy, stride, pad, cover_all):
    """ConvGradWeight with other than two spatial axes: one plain kernel with the native composition's arithmetic."""
    n = x.ndim - 2
    if x.ndim < 2 or gy.ndim != x.ndim or len(w_shape) != x.ndim:
        raise _lib.DimensionError('x, gy and w need the same number of dimensions')
    stride, pad = _pair(stride, n), _pair(pad, n)
    dims = tuple(conv_out_dim(x.shape[2 + d], w_shape[2 + d], stride[d], pad[d], cover_all) for d in range(n))
    if gy.shape != (x.shape[0], w_shape[0]) + dims or w_shape[1] != x.shape[1]:
        raise _lib.DimensionError('gy has the wrong shape')
    wdt = numpy.dtype(w_dtype)
    if _kind(wdt) != 3:
        raise _lib.DtypeError('the gradient with respect to the filters needs a floating point dtype')
    gw = ndarray.empty(tuple(w_shape), wdt)
    _lib.call('hipcx_conv_grad_weight', x.astype(wdt, False).desc(), gy.astype(wdt, False).desc(), _i64(stride), _i64(pad),
              int(bool(cover_all)), gw.desc(), ctypes.c_void_p(0), 0, current_stream())
    return gw


def conv_grad_weight(w_dtype, w_shape, x, gy, stride=1, pad=0, cover_all=False):
    """ConvGradWeightKernel after the native backend (CX/native/native_device/conv.cc:91-124): Im2Col(x), then TensorDot(gy, col)
    over the batch and the output positions -> gw[K, C, kh, kw].  The same two matrices meet in the same Dot; only the col is
    laid out [C, kh, kw, N, oh, ow] so that both Dot operands have the reduction index (n, oh, ow) as their unit-stride axis
    (the MFMA kernel's layout) and no transposed copy of the col is needed (134 against 246 us for a 3x3 layer of 256 channels)."""
    if x.ndim != 4:
        return _conv_grad_weight_nd(w_dtype, w_shape, x, gy, stride, pad, cover_all)
    (kh, kw), (sh, sw), (ph, pw) = tuple(w_shape[2:]), _pair(stride), _pair(pad)
    n, c, h, w = x.shape
    oh = conv_out_dim(h, kh, sh, ph, cover_all)
    ow = conv_out_dim(w, kw, sw, pw, cover_all)
    if gy.shape != (n, w_shape[0], oh, ow):
        raise _lib.DimensionError('gy has the wrong shape')
    wdt = numpy.dtype(w_dtype)
    if not COMPOSE_CONV_GRAD_WEIGHT and _kind(wdt) == 3 and tuple(w_shape[:2]) == (gy.shape[1], c):
        # one entry: Im2Col and the gy transpose as one kernel each, then the matrix product
        xc, gc = x.astype(wdt, False).as_contiguous(), gy.astype(wdt, False).as_contiguous()
        gw = ndarray.empty(tuple(w_shape), wdt)
        st, pd = _i64((sh, sw)), _i64((ph, pw))
        nbytes = _lib.load().hipcx_conv_grad_weight_workspace_size(xc.desc(), gc.desc(), gw.desc(), st, pd, int(bool(cover_all)))
        ws, wsp = _workspace(nbytes)
        _lib.call('hipcx_conv_grad_weight', xc.desc(), gc.desc(), st, pd, int(bool(cover_all)), gw.desc(), wsp, nbytes, current_stream())
        return gw
    xp = zeros((n, c, h + 2 * ph + (sh - 1 if cover_all else 0), w + 2 * pw + (sw - 1 if cover_all else 0)), x.dtype)
    _copy_into(xp[:, :, ph:ph + h, pw:pw + w], x)
    col_t = ndarray.empty((c, kh, kw, n, oh, ow), x.dtype)
    for r in range(kh):
        for q in range(kw):
            _copy_into(col_t[:, r, q], xp[:, :, r:r + sh * oh:sh, q:q + sw * ow:sw].transpose((1, 0, 2, 3)))
    gy_t = gy.transpose((1, 0, 2, 3)).reshape((w_shape[0], n * oh * ow))
    gw = dot(gy_t, col_t.reshape((c * kh * kw, n * oh * ow)).T, w_dtype)
    return gw.reshape(tuple(w_shape))


# True: ConvTranspose always runs as the native backend's TensorDot + Col2Im composition.
COMPOSE_CONV_TRANSPOSE = False
# True: the route (flipped convolution / scattered 1x1 convolution / composition) is chosen and issued from here, kernel call by
# kernel call, instead of inside hipcx_conv_transpose.
ROUTE_CONV_TRANSPOSE_HERE = False


def _conv_transpose_nd(x, w, b, stride, pad, out_size, out_dtype):
    """ConvTranspose with other than two spatial axes (the native kernel takes any number, CX/native/native_device/conv.cc:126-160):
    one plain kernel that adds up, per output position, what Col2Im would add there, in its order."""
    n = x.ndim - 2
    if x.ndim < 2 or w.ndim != x.ndim:
        raise _lib.DimensionError('Mismatched number of dimensions in input %r and weights %r.' % (x.shape, w.shape))
    stride, pad = _pair(stride, n), _pair(pad, n)
    if w.shape[0] != x.shape[1]:
        raise _lib.DimensionError('Mismatched number of input channels in input of shape %r and filter of shape %r' % (x.shape, w.shape))
    ksize = tuple(w.shape[2:])
    if out_size is None:
        out_size = tuple(st * (d - 1) + k - 2 * p for d, k, st, p in zip(x.shape[2:], ksize, stride, pad))
    else:
        out_size = _pair(out_size, n)
        for d, o, k, st, p in zip(x.shape[2:], out_size, ksize, stride, pad):
            if d != conv_out_dim(o, k, st, p, False) and d != conv_out_dim(o, k, st, p, True):
                raise _lib.DimensionError('Output dims %r is incosistent.' % (out_size,))
    if b is not None and (b.ndim != 1 or b.shape[0] != w.shape[1]):
        raise _lib.DimensionError('Mismatched bias shape %r for weights %r.' % (b.shape, w.shape))
    dt = numpy.dtype(out_dtype) if out_dtype is not None else (result_type(x, w, b) if b is not None else result_type(x, w))
    if _kind(dt) != 3:
        raise _lib.DtypeError('conv_transpose over %d spatial axes needs a floating point dtype' % n)
    out = ndarray.empty((x.shape[0], w.shape[1]) + tuple(out_size), dt)
    bc = b.astype(dt, False) if b is not None else None
    _lib.call('hipcx_conv_transpose', x.astype(dt, False).desc(), w.astype(dt, False).desc(), bc.desc() if bc is not None else None,
              _i64(stride), _i64(pad), out.desc(), ctypes.c_void_p(0), 0, current_stream())
    return out


def conv_transpose(x, w, b=None, stride=1, pad=0, out_size=None, out_dtype=None):
    """ConvTranspose (CX/routines/connection.cc:214-320) over the native kernel (CX/native/native_device/conv.cc:126-160):
    col = TensorDot(w, x) over the input channels, batch axis rolled first, Col2Im, bias added in place.  w: [C_in, C_out, kh, kw]."""
    if x.ndim != 4:
        return _conv_transpose_nd(x, w, b, stride, pad, out_size, out_dtype)
    stride, pad = _pair(stride), _pair(pad)
    if w.shape[0] != x.shape[1]:
        raise _lib.DimensionError('Mismatched number of input channels in input of shape %r and filter of shape %r' % (x.shape, w.shape))
    kh, kw = w.shape[2:]
    if out_size is None:  # GetConvTransposeOutDim with cover_all = false (CX/routines/connection.cc:51-56)
        out_size = tuple(st * (d - 1) + k - 2 * p for d, k, st, p in zip(x.shape[2:], (kh, kw), stride, pad))
    else:
        out_size = _pair(out_size)
        for d, o, k, st, p in zip(x.shape[2:], out_size, (kh, kw), stride, pad):
            if d != conv_out_dim(o, k, st, p, False) and d != conv_out_dim(o, k, st, p, True):
                raise _lib.DimensionError('Output dims %r is incosistent.' % (out_size,))
    dt = numpy.dtype(out_dtype) if out_dtype is not None else (result_type(x, w, b) if b is not None else result_type(x, w))
    if not COMPOSE_CONV_TRANSPOSE and not ROUTE_CONV_TRANSPOSE_HERE and _kind(dt) == 3:
        # one entry: it picks the flipped forward convolution, the scattered 1x1 convolution or the native composition itself
        xc, wc = x.astype(dt, False), w.astype(dt, False)
        bc = b.astype(dt, False) if b is not None else None
        out = ndarray.empty((x.shape[0], w.shape[1]) + tuple(out_size), dt)
        st, pd = _i64(stride), _i64(pad)
        nbytes = _lib.load().hipcx_conv_transpose_workspace_size(xc.desc(), wc.desc(), st, pd, out.desc())
        ws, wsp = _workspace(nbytes)
        _lib.call('hipcx_conv_transpose', xc.desc(), wc.desc(), bc.desc() if bc is not None else None, st, pd, out.desc(), wsp, nbytes,
                  current_stream())
        return out
    if (not COMPOSE_CONV_TRANSPOSE and stride == (1, 1) and pad[0] <= kh - 1 and pad[1] <= kw - 1 and _kind(dt) == 3
            and tuple(out_size) == tuple(d - 1 + k - 2 * p for d, k, p in zip(x.shape[2:], (kh, kw), pad))):
        # At stride 1 the transposed convolution is a forward convolution with the filters flipped in both spatial axes, their
        # channel axes swapped and the padding k - 1 - p: one MFMA convolution instead of Dot + kh*kw strided additions.  The
        # sums run in another order than the composition's (float accumulation, one rounding), equal to tolerance.
        w_flipped = w[:, :, ::-1, ::-1].transpose((1, 0, 2, 3)).copy()
        return conv(x, w_flipped, b, 1, (kh - 1 - pad[0], kw - 1 - pad[1]), False, dt)
    n, ci, h, wd = x.shape
    if not COMPOSE_CONV_TRANSPOSE and (kh, kw) == (1, 1) and pad == (0, 0) and _kind(dt) == 3 and x.size > 0:
        # A 1x1 filter at any stride: every input pixel lands on exactly one output pixel (Col2Im adds one strided plane into
        # zeros), so the result is a 1x1 forward convolution with the channel axes of w swapped, scattered to every stride-th
        # pixel of a zero-filled output.
        y1 = conv(x, w.transpose((1, 0, 2, 3)).copy(), None, 1, 0, False, dt)
        out = zeros((n, w.shape[1]) + tuple(out_size), dt)
        view = out[:, :, ::stride[0], ::stride[1]]
        hh, ww = _py.min(h, view.shape[2]), _py.min(wd, view.shape[3])  # cover_all sizes: the last input row / column falls outside
        _lib.call('hipcx_copy', y1[:, :, :hh, :ww].desc(), view[:, :, :hh, :ww].desc(), current_stream())
        if b is not None:
            bb = b.astype(dt, False).reshape((1, -1, 1, 1)).broadcast_to(out.shape)
            _lib.call('hipcx_add', out.desc(), bb.desc(), out.desc(), current_stream())
        return out
    # TensorDot(w, x) over the input channels; x goes in channels-last so that both Dot operands have the reduction index as
    # their unit-stride axis
    w2 = w.transpose((1, 2, 3, 0)).reshape((w.shape[1] * kh * kw, ci))
    x2 = x.transpose((0, 2, 3, 1)).reshape((n * h * wd, ci))
    col = dot(w2, x2.T, dt).reshape((w.shape[1], kh, kw, n, h, wd))   # [C_out, kh, kw, N, H, W]
    col = col.transpose((3, 0, 1, 2, 4, 5))                            # batch axis rolled to the top
    out = col2im(col, stride, pad, out_size)
    if b is not None:
        bb = b.astype(dt, False).reshape((1, -1, 1, 1)).broadcast_to(out.shape)
        _lib.call('hipcx_add', out.desc(), bb.desc(), out.desc(), current_stream())
    return out


def var(a, axis=None, keepdims=False):
    """Var (CX/routines/statistics.cc:147-154): Mean of the squared deviation from the (keepdims) Mean."""
    axes = _sorted_axes(axis, a.ndim)
    dt = a.dtype if _kind(a.dtype) == 3 else numpy.dtype('float32')
    diff = subtract(a.astype(dt), mean(a, axes, True))
    return mean(multiply(diff, diff), axes, keepdims)


# True: BatchNorm (training) and its gradient run as the reference's routine compositions instead of the dedicated kernels.
COMPOSE_BATCH_NORM = False


def _bn_kernel_applies(x, axes, params, same=()):
    """The dedicated kernels take a C-contiguous x of fewer than 2^31 elements reduced over every axis but 1; the per-channel arrays
    ``params`` share one dtype, x's or -- for a float16 x -- float32 (the mixed-precision call: parameters and statistics of a
    float16 network kept in float32); the arrays in ``same`` have x's dtype."""
    pd = params[0].dtype
    return (not COMPOSE_BATCH_NORM and x.ndim >= 2 and tuple(axes) == (0,) + tuple(range(2, x.ndim)) and x.is_contiguous and x.size < 2 ** 31
            and (pd == x.dtype or (x.dtype == numpy.dtype('float16') and pd == numpy.dtype('float32')))
            and _py.all(a.dtype == pd for a in params) and _py.all(a.dtype == x.dtype for a in same))


def batch_norm(x, gamma, beta, running_mean, running_var, eps=2e-5, decay=0.9, axis=None):
    """BatchNorm in training mode through GenericBatchNormKernel (CX/routines/normalization.cc:155-193): batch Mean / Var in the
    promoted dtype, ApplyGenericBatchNorm, then the running statistics are updated in place (the variance with the n/(n-1)
    correction).  Returns (out, state) with state = (x_mean, x_inv_std, beta dtype) for batch_norm_grad."""
    if _py.any(_kind(t.dtype) != 3 for t in (x, gamma, beta, running_mean, running_var)):
        raise _lib.DtypeError('BatchNorm requires floating point arrays')
    axes = _sorted_axes((0,) + tuple(range(2, x.ndim)) if axis is None else axis, x.ndim)
    red_shape = tuple(1 if i in axes else d for i, d in enumerate(x.shape))
    interm = result_type(x, gamma, beta)
    if _bn_kernel_applies(x, axes, (gamma, beta, running_mean, running_var)) and x.size > 0:
        # the dedicated kernels: two statistics passes, a per-channel finish, one normalising pass
        out = ndarray.empty(x.shape, x.dtype)
        x_mean = ndarray.empty(red_shape, interm)  # the state has the promoted dtype (CX/routines/normalization.cc:141-150)
        inv_std = ndarray.empty(red_shape, interm)
        ax = (ctypes.c_int8 * len(axes))(*axes)
        nbytes = _lib.load().hipcx_batch_norm_workspace_size(x.desc(), ax, len(axes))
        ws, wsp = _workspace(nbytes)
        _lib.call('hipcx_batch_norm', x.desc(), gamma.reshape(red_shape).desc(), beta.reshape(red_shape).desc(),
                  running_mean.reshape(red_shape).desc(), running_var.reshape(red_shape).desc(), _lib.make_scalar(float(eps)),
                  _lib.make_scalar(float(decay)), ax, len(axes), out.desc(), x_mean.desc(), inv_std.desc(), wsp, nbytes, current_stream())
        return out, (x_mean, inv_std, beta.dtype)
    xc = x.astype(interm, False)
    x_mean = mean(xc, axes, True)
    x_var = var(xc, axes, True)
    g, bt = gamma.reshape(red_shape).astype(interm, False), beta.reshape(red_shape).astype(interm, False)
    inv_std = reciprocal(sqrt(add(x_var, eps)))
    out = add(multiply(multiply(subtract(xc, x_mean), inv_std), g), bt).astype(x.dtype, False)
    n = _prod(x.shape) // _py.max(1, _prod(gamma.shape))
    inv_decay = 1.0 - float(decay)
    rm, rv = running_mean.reshape(red_shape), running_var.reshape(red_shape)
    multiply(rm, decay, out=rm)
    add(rm, multiply(x_mean, inv_decay).astype(rm.dtype, False), out=rm)
    multiply(rv, decay, out=rv)
    add(rv, multiply(x_var, inv_decay * (float(n) / _py.max(n - 1, 1))).astype(rv.dtype, False), out=rv)
    return out, (x_mean, inv_std, beta.dtype)


def batch_norm_grad(x, gamma, gout, state, axis=None):
    """GenericBatchNormGradKernel (CX/routines/normalization.cc:195-250): returns (gx, ggamma, gbeta)."""
    x_mean, x_inv_std, beta_dtype = state
    axes = _sorted_axes((0,) + tuple(range(2, x.ndim)) if axis is None else axis, x.ndim)
    red_shape = tuple(1 if i in axes else d for i, d in enumerate(x.shape))
    interm = x_mean.dtype
    if (_bn_kernel_applies(x, axes, (gamma, x_mean, x_inv_std), (gout,)) and gout.shape == x.shape and gout.is_contiguous
            and numpy.dtype(beta_dtype) == gamma.dtype and x.size > 0):
        gx = ndarray.empty(x.shape, x.dtype)
        ggamma = ndarray.empty(gamma.shape, gamma.dtype)
        gbeta = ndarray.empty(gamma.shape, gamma.dtype)
        ax = (ctypes.c_int8 * len(axes))(*axes)
        nbytes = _lib.load().hipcx_batch_norm_workspace_size(x.desc(), ax, len(axes))
        ws, wsp = _workspace(nbytes)
        _lib.call('hipcx_batch_norm_grad', x.desc(), gamma.reshape(red_shape).desc(), gout.desc(), x_mean.reshape(red_shape).desc(),
                  x_inv_std.reshape(red_shape).desc(), ax, len(axes), gx.desc(), ggamma.reshape(red_shape).desc(),
                  gbeta.reshape(red_shape).desc(), wsp, nbytes, current_stream())
        return gx, ggamma, gbeta
    n = _prod(x.shape) // _py.max(1, _prod(gamma.shape))
    inv_n = 1.0 / n
    gc = gout.astype(interm, False)
    x_hat = multiply(subtract(x.astype(interm, False), x_mean), x_inv_std)
    ggamma = sum(multiply(gc, x_hat), axes, True)
    gbeta = sum(gc, axes, True)
    g = gamma.reshape(red_shape).astype(interm, False)
    gx = multiply(multiply(g, x_inv_std), subtract(gc, multiply(add(multiply(x_hat, ggamma), gbeta), inv_n)))
    return (gx.astype(x.dtype, False), ggamma.astype(gamma.dtype, False).reshape(gamma.shape),
            gbeta.astype(beta_dtype, False).reshape(gamma.shape))


# True: pooling gradients run as the native backend's Im2Col / ArgMax / Col2Im composition instead of the dedicated kernels (tests
# compare the two bit for bit).
COMPOSE_POOL_GRADIENTS = False


def _pool_grad_nd(entry, x, gout, ksize, stride, pad, flag):
    """MaxPoolGrad / AveragePoolGrad with other than two spatial axes: one plain kernel per call, the bits of the native composition.
    `flag`: cover_all for max pooling, the pad mode for average pooling (whose output extents never use cover_all)."""
    n = x.ndim - 2
    is_max = entry == 'hipcx_max_pool_grad'
    if n < 1 or gout.ndim != x.ndim or gout.dtype != x.dtype:
        raise _lib.DimensionError('gout needs the rank and dtype of x (at least one spatial axis)')
    if x.dtype == numpy.dtype('bool') or (not is_max and _kind(x.dtype) != 3):
        raise _lib.DtypeError('pooling gradient: unsupported dtype %s' % x.dtype)
    ksize = _pair(ksize, n)
    stride = ksize if stride is None else _pair(stride, n)
    pad = _pair(pad, n)
    dims = tuple(conv_out_dim(x.shape[2 + d], ksize[d], stride[d], pad[d], bool(flag) if is_max else False) for d in range(n))
    if gout.shape != tuple(x.shape[:2]) + dims:
        raise _lib.DimensionError('gout has the wrong shape')
    gx = ndarray.empty(x.shape, x.dtype)
    if is_max:
        _lib.call(entry, x.desc(), gout.desc(), _i64(ksize), _i64(stride), _i64(pad), flag, gx.desc(), ctypes.c_void_p(0), 0, current_stream())
    else:
        _lib.call(entry, gout.desc(), _i64(ksize), _i64(stride), _i64(pad), flag, gx.desc(), current_stream())
    return gx


def max_pool_grad(x, gout, ksize, stride=None, pad=0, cover_all=False):
    """MaxPoolGradKernel after the native backend (CX/native/native_device/pool.cc:97-143): Im2Col with -inf padding, ArgMax over
    the kernel axes (its tie rule picks the position), gout placed at that kernel offset of an otherwise zero col, Col2Im."""
    if x.ndim != 4:
        return _pool_grad_nd('hipcx_max_pool_grad', x, gout, ksize, stride, pad, int(bool(cover_all)))
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    if x.ndim == 4 and x.dtype != numpy.dtype('bool') and gout.dtype == x.dtype and not COMPOSE_POOL_GRADIENTS:
        # one kernel: every input position gathers, in kernel-offset order, gout of the windows whose ArgMax it is -- the bits
        # of the composition below
        oh = conv_out_dim(x.shape[2], ksize[0], stride[0], pad[0], cover_all)
        ow = conv_out_dim(x.shape[3], ksize[1], stride[1], pad[1], cover_all)
        if gout.shape != (x.shape[0], x.shape[1], oh, ow):
            raise _lib.DimensionError('gout has the wrong shape')
        gx = ndarray.empty(x.shape, x.dtype)
        nbytes = _lib.load().hipcx_max_pool_grad_workspace_size(gout.desc())
        ws, wsp = _workspace(nbytes)
        _lib.call('hipcx_max_pool_grad', x.desc(), gout.desc(), _i64(ksize), _i64(stride), _i64(pad), int(bool(cover_all)), gx.desc(),
                  wsp, nbytes, current_stream())
        return gx
    lowest = -numpy.inf if _kind(x.dtype) == 3 else (0 if x.dtype == numpy.dtype('bool') else int(numpy.iinfo(x.dtype).min))
    col = im2col(x, ksize, stride, pad, cover_all, lowest)            # [N, C, kh, kw, oh, ow]
    indices = argmax(col, (2, 3))                                     # [N, C, oh, ow]
    if indices.shape != gout.shape:
        raise _lib.DimensionError('gout has the wrong shape')
    # Every output position owns its own kt slots of the flat col, so the reference's AddAt at (index + offset) writes each
    # slot at most once: the same values come out of a select against the kernel offsets, which runs in parallel.
    taps = arange(0, ksize[0] * ksize[1], 1, dtype='int64').reshape((1, 1) + ksize + (1, 1))
    n, c, oh, ow = gout.shape
    full_shape = (n, c) + ksize + (oh, ow)
    hit = equal(indices.reshape((n, c, 1, 1, oh, ow)).broadcast_to(full_shape), taps.broadcast_to(full_shape))
    gcol = where(hit, gout.reshape((n, c, 1, 1, oh, ow)).broadcast_to(full_shape), 0)
    return col2im(gcol, stride, pad, x.shape[2:])


def max_pool_grad_grad(x, ggx, ksize, stride=None, pad=0, cover_all=False):
    """MaxPoolGradGradKernel after the native backend (CX/native/native_device/pool.cc:147-177): the element of every window
    of ggx at the position where x had its maximum -- Im2Col(ggx) with the kernel axes last, flattened, Take at index + offset."""
    if x.ndim != 4:
        n = x.ndim - 2
        if n < 1 or ggx.shape != x.shape or ggx.dtype != x.dtype or x.dtype == numpy.dtype('bool'):
            raise _lib.DimensionError('ggx needs the shape and dtype of x (at least one spatial axis, not bool)')
        ksize = _pair(ksize, n)
        stride = ksize if stride is None else _pair(stride, n)
        pad = _pair(pad, n)
        dims = tuple(conv_out_dim(x.shape[2 + d], ksize[d], stride[d], pad[d], cover_all) for d in range(n))
        ggout = ndarray.empty(tuple(x.shape[:2]) + dims, x.dtype)
        _lib.call('hipcx_max_pool_grad_grad', x.desc(), ggx.desc(), _i64(ksize), _i64(stride), _i64(pad), int(bool(cover_all)),
                  ggout.desc(), current_stream())
        return ggout
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    if x.ndim == 4 and x.dtype != numpy.dtype('bool') and ggx.dtype == x.dtype and ggx.shape == x.shape and not COMPOSE_POOL_GRADIENTS:
        oh = conv_out_dim(x.shape[2], ksize[0], stride[0], pad[0], cover_all)
        ow = conv_out_dim(x.shape[3], ksize[1], stride[1], pad[1], cover_all)
        ggout = ndarray.empty((x.shape[0], x.shape[1], oh, ow), x.dtype)
        _lib.call('hipcx_max_pool_grad_grad', x.desc(), ggx.desc(), _i64(ksize), _i64(stride), _i64(pad), int(bool(cover_all)),
                  ggout.desc(), current_stream())
        return ggout
    lowest = -numpy.inf if _kind(x.dtype) == 3 else (0 if x.dtype == numpy.dtype('bool') else int(numpy.iinfo(x.dtype).min))
    indices = argmax(im2col(x, ksize, stride, pad, cover_all, lowest), (2, 3))
    kt = ksize[0] * ksize[1]
    total = _prod(indices.shape)
    offset = arange(0, total * kt, kt, dtype='int64').reshape(indices.shape)
    col = im2col(ggx, ksize, stride, pad, cover_all, lowest).transpose((0, 1, 4, 5, 2, 3))
    return take(col.reshape((total * kt,)), add(indices, offset), 0, 'raise')


def average_pool_grad(x, gout, ksize, stride=None, pad=0, pad_mode='ignore'):
    """AveragePoolGradKernel as the native backend runs it (CX/native/native_device/pool.cc:304-346): gout (divided by the
    per-window width first in 'ignore' mode) broadcast over the kernel axes, Col2Im, and in 'zero' mode a division by the
    window size afterwards."""
    if x.ndim != 4:
        return _pool_grad_nd('hipcx_average_pool_grad', x, gout, ksize, stride, pad, {'zero': 1, 'ignore': 2}[pad_mode])
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    n, c, oh, ow = gout.shape
    if x.ndim == 4 and _kind(x.dtype) == 3 and gout.dtype == x.dtype and not COMPOSE_POOL_GRADIENTS:
        gx = ndarray.empty(x.shape, x.dtype)
        _lib.call('hipcx_average_pool_grad', gout.desc(), _i64(ksize), _i64(stride), _i64(pad), {'zero': 1, 'ignore': 2}[pad_mode],
                  gx.desc(), current_stream())
        return gx
    g = gout
    if pad_mode == 'ignore':
        def widths(dim, k, st, p, count):  # GetPadModeIgnorePoolingWidths (pool.cc:197-250)
            return numpy.array([_py.min(i * st - p + k, dim) - _py.max(i * st - p, 0) for i in range(count)], x.dtype)
        wi = numpy.outer(widths(x.shape[2], ksize[0], stride[0], pad[0], oh), widths(x.shape[3], ksize[1], stride[1], pad[1], ow))
        g = divide(gout, array(wi.astype(x.dtype)))
    gcol = g.reshape((n, c, 1, 1, oh, ow)).broadcast_to((n, c, ksize[0], ksize[1], oh, ow))
    gx = col2im(gcol, stride, pad, x.shape[2:])
    if pad_mode == 'zero':
        gx = gx.copy()
        _lib.call('hipcx_divide_as', gx.desc(), _lib.make_scalar(ksize[0] * ksize[1]), gx.desc(), current_stream())
    return gx


# ---------------------------------------------------------------------------------------------
# composite routines
# ---------------------------------------------------------------------------------------------
def lstm(c, x):
    """Lstm cell (CX/routines/connection.cc:396-446), equal batch sizes: gates are stride-4 views of x."""
    if x.shape[0] > c.shape[0]:
        raise _lib.DimensionError('The batch size of x must be equal to or less than the size of c')
    if x.shape[1] != 4 * c.shape[1]:
        raise _lib.DimensionError('Expected dimension at axis 1 of x to be equal 4 times dimension at axis 1 of c.')
    if _kind(c.dtype) != 3:
        raise _lib.DtypeError('Expected data type float')
    if c.dtype != x.dtype:
        raise _lib.DtypeError('Datatypes of c and x should be equal')
    if x.shape[0] != c.shape[0]:
        raise _lib.ChainerxNotImplementedError('ragged batches are not on the supported path')
    xr = x.reshape((x.shape[0], x.shape[1] // 4, 4) + tuple(x.shape[2:]))
    gates = [g.squeeze(2) for g in split(xr, 4, 2)]
    a = tanh(gates[0])
    i = sigmoid(gates[1])
    f = sigmoid(gates[2])
    o = sigmoid(gates[3])
    new_c = add(multiply(a, i), multiply(f, c))
    h = multiply(o, tanh(new_c))
    return h, new_c


def lstm_fused(c, x):
    """Opt-in: the Lstm cell through hipcx_lstm_cell -- one kernel instead of ~25; same checks and errors as lstm."""
    if c.ndim != 2 or x.ndim != 2:
        return lstm(c, x)
    h = ndarray.empty(c.shape, c.dtype)
    new_c = ndarray.empty(c.shape, c.dtype)
    _lib.call('hipcx_lstm_cell', c.desc(), x.desc(), h.desc(), new_c.desc(), current_stream())
    return h, new_c


def stack(arrays, axis=0):
    """Stack = Empty + one CopyKernel per input into a view of the new axis (CX/routines/manipulation.cc Stack)."""
    arrays = list(arrays)
    if not arrays:
        raise _lib.DimensionError('Need at least one array to stack')
    first = arrays[0]
    axis = _normalize_axis(axis, first.ndim + 1)
    dtype = first.dtype
    for a in arrays:
        if a.shape != first.shape:
            raise _lib.DimensionError('All arrays need to have the same shape')
        dtype = promote_types(dtype, a.dtype)
    out = ndarray.empty(first.shape[:axis] + (len(arrays),) + first.shape[axis:], dtype)
    for i, a in enumerate(arrays):
        key = [slice(None)] * out.ndim
        key[axis] = i
        _lib.call('hipcx_copy', a.desc(), out[tuple(key)].desc(), current_stream())
    return out


def clipped_relu(x, z):
    """ClippedRelu = Minimum(Maximum(0, x), z) (CX/routines/activation.cc:51-55)."""
    return minimum(maximum(x.astype(_math_result_dtype(x.dtype), False), 0), z)


def crelu(x, axis=1):
    """CRelu = Relu(Concatenate({x, -x}, axis)) (CX/routines/activation.cc:57-64)."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    return relu(concatenate([xc, negative(xc)], axis))


def elu(x, alpha=1.0):
    """Elu = Where(x > 0, x, alpha * Expm1(x)) (CX/routines/activation.cc:66-72)."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    return where(greater(xc, zeros((), xc.dtype)), xc, multiply(expm1(xc), alpha))


def leaky_relu(x, slope=0.2):
    """LeakyRelu = Where(x >= 0, x, slope * x) (CX/routines/activation.cc:86-92)."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    return where(greater_equal(xc, zeros((), xc.dtype)), xc, multiply(xc, slope))


def softplus(x, beta=1.0):
    """Softplus = (Maximum(beta*x, 0) + Log1p(Exp(-Fabs(beta*x)))) / beta (CX/routines/activation.cc:151-158)."""
    xc = x.astype(_math_result_dtype(x.dtype), False)
    bx = multiply(xc, beta)
    return multiply(add(maximum(bx, 0), log1p(exp(negative(fabs(bx))))), 1.0 / beta)


def _extract_gates(x, n_splits, axis):
    """ExtractGates (CX/routines/activation.cc:30-46): axis 1 -> [B, n, H] (gate-major), axis 2 -> [B, H, n] (unit-major)."""
    rest = tuple(x.shape[2:])
    if axis == 1:
        xr = x.reshape((x.shape[0], n_splits, x.shape[1] // n_splits) + rest)
    else:
        xr = x.reshape((x.shape[0], x.shape[1] // n_splits, n_splits) + rest)
    return [g.squeeze(axis) for g in split(xr, n_splits, axis)]


def tree_lstm(*arrays):
    """TreeLstm(c_1..c_n, x) -> (c, h); gates of x are gate-major: a, i, o, f_1..f_n (CX/routines/activation.cc:94-121)."""
    arrays = list(arrays)
    n_ary = len(arrays) - 1
    gates = _extract_gates(arrays[-1], 3 + n_ary, 1)
    a = tanh(gates[0])
    i = sigmoid(gates[1])
    o = sigmoid(gates[2])
    fs = [sigmoid(f) for f in gates[3:]]
    acc = multiply(arrays[0], fs[0])
    for k in range(1, n_ary):
        acc = add(acc, multiply(arrays[k], fs[k]))
    c = add(multiply(a, i), acc)
    h = multiply(o, tanh(c))
    return c, h


def slstm(c_prev1, c_prev2, x1, x2):
    """SLstm -> (c, h); gates are unit-major a, i, f, o (CX/routines/activation.cc:123-149)."""
    a1, i1, f1, o1 = _extract_gates(x1, 4, 2)
    a2, i2, f2, o2 = _extract_gates(x2, 4, 2)
    a1, i1, f1 = tanh(a1), sigmoid(i1), sigmoid(f1)
    a2, i2, f2 = tanh(a2), sigmoid(i2), sigmoid(f2)
    o = sigmoid(add(o1, o2))
    c = add(add(add(multiply(a1, i1), multiply(a2, i2)), multiply(f1, c_prev1)), multiply(f2, c_prev2))
    h = multiply(o, tanh(c))
    return c, h


# ---------------------------------------------------------------------------------------------
# n-step recurrent networks: the composition every backend but cuDNN's runs (CX/routines/n_step_rnn.cc:360-429)
# ---------------------------------------------------------------------------------------------
def _stack_weight(ws):
    """StackWeight (CX/routines/n_step_rnn.cc:41-54): row u*len(ws) + g of the result is row u of ws[g]."""
    w = stack(ws, 1)
    return w.reshape((w.shape[0] * w.shape[1],) + tuple(w.shape[2:]))


def _gru_impl(x, h, c, ws, bs, activation):
    xw = concatenate([ws[0], ws[1], ws[2]], 0)
    hw = concatenate([ws[3], ws[4], ws[5]], 0)
    xb = concatenate([bs[0], bs[1], bs[2]], 0)
    hb = concatenate([bs[3], bs[4], bs[5]], 0)
    gx = split(linear(x, xw, xb), 3, 1)
    gh = split(linear(h, hw, hb), 3, 1)
    r = sigmoid(add(gx[0], gh[0]))
    z = sigmoid(add(gx[1], gh[1]))
    h_bar = tanh(add(gx[2], multiply(r, gh[2])))
    return [add(multiply(subtract(1, z), h_bar), multiply(z, h))]


def _lstm_impl(x, h, c, ws, bs, activation, cell=None):
    xw = _stack_weight([ws[2], ws[0], ws[1], ws[3]])
    hw = _stack_weight([ws[6], ws[4], ws[5], ws[7]])
    xb = _stack_weight([bs[2], bs[0], bs[1], bs[3]])
    hb = _stack_weight([bs[6], bs[4], bs[5], bs[7]])
    lstm_in = add(linear(x, xw, xb), linear(h, hw, hb))
    return list((cell or lstm)(c, lstm_in))


def _lstm_impl_fused(x, h, c, ws, bs, activation):
    return _lstm_impl(x, h, c, ws, bs, activation, cell=lstm_fused)


def _rnn_impl(x, h, c, ws, bs, activation):
    rnn_in = add(linear(x, ws[0], bs[0]), linear(h, ws[1], bs[1]))
    return [tanh(rnn_in) if activation == 'tanh' else relu(rnn_in)]


def _lstm_direction_fused(xs, h, c, ws, bs):
    """One layer and direction of an LSTM with the loop-invariant work hoisted (opt-in): the gate rows are stacked once instead of
    once per time step, the input projection of all time steps is one Dot over the concatenated batch, and each step is
    Dot(h, hw) + Add + one hipcx_lstm_cell call.  State rows beyond a step's batch keep their values, as in the composed loop."""
    h = h.reshape((h.shape[1], h.shape[2]))
    c = c.reshape(h.shape)
    xw = _stack_weight([ws[2], ws[0], ws[1], ws[3]])
    hw = _stack_weight([ws[6], ws[4], ws[5], ws[7]])
    xb = _stack_weight([bs[2], bs[0], bs[1], bs[3]])
    hb = _stack_weight([bs[6], bs[4], bs[5], bs[7]])
    sizes = [x.shape[0] for x in xs]
    if _py.max(sizes) > h.shape[0]:
        raise _lib.DimensionError('The batch size of x must be equal to or less than the size of state')
    gx_all = linear(concatenate(xs, 0) if len(xs) > 1 else xs[0], xw, xb)
    h_list = []
    pos = 0
    for n in sizes:
        gx = gx_all[pos:pos + n]
        pos += n
        full = n == h.shape[0]
        h_n, c_n = lstm_fused(c if full else c[:n], add(gx, linear(h if full else h[:n], hw, hb)))
        h_list.append(h_n)
        if full:
            h, c = h_n, c_n
        else:
            h = concatenate([h_n, h[n:]], 0)
            c = concatenate([c_n, c[n:]], 0)
    return [h, c], h_list


def _one_directional_loop(impl, xs, h, c, ws, bs, activation):
    if impl is _lstm_impl_fused:
        return _lstm_direction_fused(xs, h, c, ws, bs)
    h = h.reshape((h.shape[1], h.shape[2]))
    if c is not None:
        c = c.reshape(h.shape)
    h_list = []
    for x in xs:
        if x.shape[0] > h.shape[0]:
            raise _lib.DimensionError('The batch size of x must be equal to or less than the size of state')
        h_split = split(h, [x.shape[0], h.shape[0]], 0)
        if c is not None:
            c_split = split(c, [x.shape[0], c.shape[0]], 0)
            h_c = impl(x, h_split[0], c_split[0], ws, bs, activation)
            c_split[0] = h_c[1]
            c = concatenate(c_split, 0)
        else:
            h_c = impl(x, h_split[0], None, ws, bs, activation)
        h_list.append(h_c[0])
        h_split[0] = h_c[0]
        h = concatenate(h_split, 0)
    return ([h] if c is None else [h, c]), h_list


def _n_step_rnn_impl(impl, n_layers, hx, cx, ws, bs, xs, bidirectional, activation=None):
    direction = 2 if bidirectional else 1
    hx_list = split(hx, hx.shape[0], 0)
    cx_list = split(cx, cx.shape[0], 0) if cx is not None else [None] * hx.shape[0]
    xs_next = list(xs)
    hy, cy = [], []
    for layer in range(n_layers):
        xs = xs_next
        idx = direction * layer
        state, h_forward = _one_directional_loop(impl, xs, hx_list[idx], cx_list[idx], ws[idx], bs[idx], activation)
        hy.append(state[0])
        if cx is not None:
            cy.append(state[1])
        if bidirectional:
            idx += 1
            state, h_backward = _one_directional_loop(impl, xs[::-1], hx_list[idx], cx_list[idx], ws[idx], bs[idx], activation)
            h_backward = h_backward[::-1]
            xs_next = [concatenate([f, b], 1) for f, b in zip(h_forward, h_backward)]
            hy.append(state[0])
            if cx is not None:
                cy.append(state[1])
        else:
            xs_next = h_forward
    if cx is not None:
        return stack(hy, 0), stack(cy, 0), xs_next
    return stack(hy, 0), xs_next


def _descriptor_pointers(arrays):
    """A C array of hipcx_array pointers for `arrays` (the arrays must stay alive while it is used)."""
    for a in arrays:
        a.desc()  # builds and caches the descriptor
    return (ctypes.POINTER(_lib.CArray) * len(arrays))(*[ctypes.pointer(a._desc) for a in arrays])


class RnnGradState(object):
    """What RnnKernel hands to RnnBackwardKernel (chainerx::RnnGradState, CX/kernels/rnn.h:22-32): the reserve the forward pass
    filled and the call's arguments."""

    def __init__(self, **kw):
        self.__dict__.update(kw)


_RNN_MODES = {'gru': 0, 'lstm': 1, 'rnn': 2}


def rnn(n_layers, hx, cx, ws, bs, xs, bidirectional, mode, activation=None, training=False):
    """RnnKernel::Call (CX/kernels/rnn.h:34-49) through hipcx_n_step_rnn, float32: ``mode`` 'gru' / 'lstm' / 'rnn' (or the
    reference's 0 / 1 / 2), ``activation`` 'tanh' / 'relu' for 'rnn'.  ws[layer * directions + direction] / bs[...] hold the 6 / 8 / 2
    matrices / vectors of that layer and direction.  Returns ((hy, cy or None), ys, state); ``state`` is None unless ``training``."""
    m = _RNN_MODES.get(mode, mode)
    if m not in (0, 1, 2):
        raise _lib.ChainerxError('rnn: unknown mode %r' % (mode,))
    act = {None: 0, 'tanh': 0, 'relu': 1}[activation]
    d = 2 if bidirectional else 1
    flat_w = [w for group in ws for w in group]
    flat_b = [b for group in bs for b in group]
    xs = list(xs)
    hy = ndarray.empty(hx.shape, hx.dtype)
    cy = ndarray.empty(cx.shape, cx.dtype) if m == 1 else None
    ys = [ndarray.empty((x.shape[0], d * hx.shape[2]), hx.dtype) for x in xs]
    pw, pb, px, py = (_descriptor_pointers(v) for v in (flat_w, flat_b, xs, ys))
    L = _lib.load()
    rbytes = L.hipcx_n_step_rnn_reserve_size(n_layers, d - 1, m, hx.desc(), px, len(xs)) if training else 0
    reserve, rp = _workspace(rbytes) if training else (None, None)
    nbytes = L.hipcx_n_step_rnn_workspace_size(n_layers, d - 1, m, int(bool(training)), hx.desc(), px, len(xs))
    wsb, wsp = _workspace(nbytes)
    _lib.call('hipcx_n_step_rnn', n_layers, d - 1, m, act, hx.desc(), cx.desc() if m == 1 else None, pw, pb, px, len(xs), hy.desc(),
              cy.desc() if m == 1 else None, py, rp, rbytes, wsp, nbytes, current_stream())
    state = None
    if training:
        state = RnnGradState(reserve=reserve, reserve_ptr=rp, reserve_bytes=rbytes, n_layers=n_layers, directions=d, mode=m, activation=act,
                             hx=hx, ws=flat_w, bs=flat_b, xs=xs)
    return (hy, cy), ys, state


def rnn_backward(state, dhy, dcy, dys):
    """RnnBackwardKernel::Call (CX/kernels/rnn.h:51-66) through hipcx_n_step_rnn_backward: the gradients of the forward pass that
    produced ``state``.  ``dcy`` and entries of ``dys`` may be None (zeros).  Returns ((dhx, dcx or None), dws, dbs, dxs) with dws / dbs
    flat in the order of the forward call's matrices."""
    st = state
    dhx = ndarray.empty(st.hx.shape, st.hx.dtype)
    dcx = ndarray.empty(st.hx.shape, st.hx.dtype) if st.mode == 1 else None
    dws = [ndarray.empty(w.shape, w.dtype) for w in st.ws]
    dbs = [ndarray.empty(b.shape, b.dtype) for b in st.bs]
    dxs = [ndarray.empty(x.shape, x.dtype) for x in st.xs]
    pw, pb, px, pdw, pdb, pdx = (_descriptor_pointers(v) for v in (st.ws, st.bs, st.xs, dws, dbs, dxs))
    for a in dys:
        if a is not None:
            a.desc()
    pdy = (ctypes.POINTER(_lib.CArray) * len(dys))(*[ctypes.pointer(a._desc) if a is not None else None for a in dys])
    nbytes = _lib.load().hipcx_n_step_rnn_workspace_size(st.n_layers, st.directions - 1, st.mode, 1, st.hx.desc(), px, len(st.xs))
    wsb, wsp = _workspace(nbytes)
    _lib.call('hipcx_n_step_rnn_backward', st.n_layers, st.directions - 1, st.mode, st.activation, st.hx.desc(), pw, pb, px, len(st.xs),
              dhy.desc(), dcy.desc() if (dcy is not None and st.mode == 1) else None, pdy, st.reserve_ptr, st.reserve_bytes, dhx.desc(),
              dcx.desc() if st.mode == 1 else None, pdw, pdb, pdx, wsp, nbytes, current_stream())
    return (dhx, dcx), dws, dbs, dxs


def _n_step_lstm_kernel(n_layers, hx, cx, ws, bs, xs):
    """The RnnKernel entry (hipcx_n_step_lstm): weights packed once, one launch per wavefront stage."""
    if len(ws) != n_layers or len(bs) != n_layers or _py.any(len(w) != 8 for w in ws) or _py.any(len(b) != 8 for b in bs):
        raise _lib.DimensionError('n_step_lstm needs eight matrices and eight biases per layer')
    flat_w = [w for layer in ws for w in layer]
    flat_b = [b for layer in bs for b in layer]
    xs = list(xs)
    hy = ndarray.empty(hx.shape, hx.dtype)
    cy = ndarray.empty(cx.shape, cx.dtype)
    ys = [ndarray.empty((x.shape[0], hx.shape[2]), hx.dtype) for x in xs]
    pw, pb, px, py = (_descriptor_pointers(v) for v in (flat_w, flat_b, xs, ys))
    nbytes = _lib.load().hipcx_n_step_lstm_workspace_size(n_layers, hx.desc(), px, len(xs))
    wsb, wsp = _workspace(nbytes)
    _lib.call('hipcx_n_step_lstm', n_layers, hx.desc(), cx.desc(), pw, pb, px, len(xs), hy.desc(), cy.desc(), py, wsp, nbytes, current_stream())
    return hy, cy, ys


def n_step_lstm(n_layers, hx, cx, ws, bs, xs, fused=False, kernel=False):
    """NStepLstm (CX/routines/n_step_rnn.cc:434-443) -> (hy, cy, ys).  ws[layer] / bs[layer] hold the eight matrices / vectors in
    cuDNN order: input, forget, cell, output for x, then the same for h.  `fused` (opt-in) runs each cell through hipcx_lstm_cell;
    `kernel` (opt-in, float32) runs the whole routine through hipcx_n_step_lstm, the RnnKernel the reference gives its cuda backend."""
    if kernel and hx.dtype == numpy.dtype('float32'):
        return _n_step_lstm_kernel(n_layers, hx, cx, ws, bs, xs)
    return _n_step_rnn_impl(_lstm_impl_fused if fused else _lstm_impl, n_layers, hx, cx, ws, bs, xs, False)


def _rnn_kernel_route(kernel, hx):
    """`kernel` (opt-in) runs a whole n-step routine through hipcx_n_step_rnn, the RnnKernel the reference gives its cuda backend
    (CX/routines/n_step_rnn.cc:210); float32 only, other dtypes take the composition."""
    return kernel and hx.dtype == numpy.dtype('float32')


def n_step_bilstm(n_layers, hx, cx, ws, bs, xs, fused=False, kernel=False):
    """NStepBiLstm (CX/routines/n_step_rnn.cc:445-454): ws[2*layer + direction]."""
    if _rnn_kernel_route(kernel, hx):
        (hy, cy), ys, _ = rnn(n_layers, hx, cx, ws, bs, xs, True, 'lstm')
        return hy, cy, ys
    return _n_step_rnn_impl(_lstm_impl_fused if fused else _lstm_impl, n_layers, hx, cx, ws, bs, xs, True)


def n_step_gru(n_layers, hx, ws, bs, xs, kernel=False):
    """NStepGru (CX/routines/n_step_rnn.cc:456-465) -> (hy, ys); six matrices per layer: reset, update, candidate for x, then h."""
    if _rnn_kernel_route(kernel, hx):
        (hy, _), ys, _ = rnn(n_layers, hx, None, ws, bs, xs, False, 'gru')
        return hy, ys
    return _n_step_rnn_impl(_gru_impl, n_layers, hx, None, ws, bs, xs, False)


def n_step_bigru(n_layers, hx, ws, bs, xs, kernel=False):
    """NStepBiGru (CX/routines/n_step_rnn.cc:467-476)."""
    if _rnn_kernel_route(kernel, hx):
        (hy, _), ys, _ = rnn(n_layers, hx, None, ws, bs, xs, True, 'gru')
        return hy, ys
    return _n_step_rnn_impl(_gru_impl, n_layers, hx, None, ws, bs, xs, True)


def n_step_rnn(n_layers, hx, ws, bs, xs, activation='tanh', kernel=False):
    """NStepRnn (CX/routines/n_step_rnn.cc:478-487) -> (hy, ys); activation 'tanh' or 'relu'."""
    if _rnn_kernel_route(kernel, hx):
        (hy, _), ys, _ = rnn(n_layers, hx, None, ws, bs, xs, False, 'rnn', activation)
        return hy, ys
    return _n_step_rnn_impl(_rnn_impl, n_layers, hx, None, ws, bs, xs, False, activation)


def n_step_birnn(n_layers, hx, ws, bs, xs, activation='tanh', kernel=False):
    """NStepBiRnn (CX/routines/n_step_rnn.cc:489-498)."""
    if _rnn_kernel_route(kernel, hx):
        (hy, _), ys, _ = rnn(n_layers, hx, None, ws, bs, xs, True, 'rnn', activation)
        return hy, ys
    return _n_step_rnn_impl(_rnn_impl, n_layers, hx, None, ws, bs, xs, True, activation)


def softmax_cross_entropy(x, t):
    """Chainer's F.softmax_cross_entropy forward for chainerx arrays with the default reduce='mean', normalize=True
    (chainer/functions/loss/softmax_cross_entropy.py:123-130): a Python-level composition, 15 kernel calls."""
    score = log_softmax(x, 1)
    mask = equal(t[:, None], arange(score.shape[1], dtype=t.dtype)).astype(score.dtype)
    return multiply(sum(multiply(score, mask)), divide(-1, sum(mask)))


# ---------------------------------------------------------------------------------------------
# operators
# ---------------------------------------------------------------------------------------------
def _install_operators():
    ndarray.__add__ = lambda self, o: add(self, o)
    ndarray.__radd__ = lambda self, o: add(self, o)
    ndarray.__sub__ = lambda self, o: subtract(self, o)
    ndarray.__rsub__ = lambda self, o: subtract(o, self)
    ndarray.__mul__ = lambda self, o: multiply(self, o)
    ndarray.__rmul__ = lambda self, o: multiply(self, o)
    ndarray.__truediv__ = lambda self, o: divide(self, o)
    ndarray.__rtruediv__ = lambda self, o: divide(o, self)
    ndarray.__neg__ = lambda self: negative(self)
    ndarray.__iadd__ = lambda self, o: add(self, o, out=self)
    ndarray.__isub__ = lambda self, o: subtract(self, o, out=self)
    ndarray.__imul__ = lambda self, o: multiply(self, o, out=self)
    ndarray.__itruediv__ = lambda self, o: divide(self, o, out=self)
    ndarray.__eq__ = lambda self, o: equal(self, o)
    ndarray.__ne__ = lambda self, o: not_equal(self, o)
    ndarray.__gt__ = lambda self, o: greater(self, o)
    ndarray.__ge__ = lambda self, o: greater_equal(self, o)
    ndarray.__hash__ = None
    ndarray.sum = lambda self, axis=None, keepdims=False: sum(self, axis, keepdims)
    ndarray.max = lambda self, axis=None, keepdims=False: amax(self, axis, keepdims)
    ndarray.argmax = lambda self, axis=None: argmax(self, axis)
    ndarray.mean = lambda self, axis=None, keepdims=False: mean(self, axis, keepdims)
    ndarray.dot = lambda self, o: dot(self, o)
    ndarray.take = lambda self, indices, axis, mode=None: take(self, indices, axis, mode)


_install_operators()

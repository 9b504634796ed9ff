"""Parity oracle: the ChainerX *native* (CPU) backend restated with numpy + ``liboracle.so``.

TEST INFRASTRUCTURE ONLY.  Importers: ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.  The product package ``chainer_amd`` never imports this.

Each function follows the reference routine + native kernel named in its docstring (paths relative
to the reference tree, ``CX/`` = ``chainerx_cc/chainerx/``), including the order of floating point
operations wherever the native backend fixes one: every elementwise op rounds to the array dtype
(float16 through float32, as ``chainerx::Float16`` does), reductions use the native pairwise tree,
Dot/Conv accumulate with one fused multiply-add per term in (i, l, j) order.

How each function is pinned (golden vectors of the reference's own tests, closed forms, brute
force) is recorded in ``tests/test_oracle_pins.py``; functions whose bit pattern only a compiled
reference run could pin say "parity unpinned (bit level)" below -- their tolerance-level behaviour
is still pinned.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'liboracle.so')
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i64p = ctypes.POINTER(ctypes.c_int64)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64 = ctypes.c_int64


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError('oracle/liboracle.so is not built: run `make -C oracle`')
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _ptr(a, ctype):
    return a.ctypes.data_as(ctype)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------------------------------------
# float16 (CX/float16.cc:27-89,161-193)
# ---------------------------------------------------------------------------------------------
def float_to_half_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_float_to_half(_ptr(x, _f32p), _ptr(out, _u16p), _i64(x.size))
    return out


def half_bits_to_float(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_half_to_float(_ptr(h, _u16p), _ptr(out, _f32p), _i64(h.size))
    return out


# ---------------------------------------------------------------------------------------------
# elementwise (CX/native/native_device/{arithmetic,exp_log,hyperbolic,misc,logic,copy,fill}.cc)
# numpy applies exactly one IEEE rounding per operation in the array dtype, float16 via float32,
# which is the native functors' arithmetic (CX/arithmetic_ops.h:7-25, CX/float16.h operators).
# ---------------------------------------------------------------------------------------------
def astype(x, dtype):
    """CopyKernel: static_cast<Out>(in) (copy.cc:21-35)."""
    with np.errstate(all='ignore'):
        return np.asarray(x).astype(dtype)


def _scalar_as(value, dtype):
    return np.asarray(value).astype(dtype)[()]


def add(x1, x2):
    x1, x2 = np.asarray(x1), np.asarray(x2)
    if x1.dtype == np.bool_ and x2.dtype == np.bool_:
        return x1 | x2
    with np.errstate(all='ignore'):
        return x1 + x2


def subtract(x1, x2):
    with np.errstate(all='ignore'):
        return np.asarray(x1) - np.asarray(x2)


def multiply(x1, x2):
    x1, x2 = np.asarray(x1), np.asarray(x2)
    if x1.dtype == np.bool_ and x2.dtype == np.bool_:
        return x1 & x2
    with np.errstate(all='ignore'):
        return x1 * x2


def divide(x1, x2):
    """DivideKernel on floats (routine TrueDivide casts ints to float32 first, CX/routines/arithmetic.cc:395-417)."""
    x1, x2 = np.asarray(x1), np.asarray(x2)
    with np.errstate(all='ignore'):
        return x1 / x2


def exp(x):
    with np.errstate(all='ignore'):
        return np.exp(x)


def log(x):
    with np.errstate(all='ignore'):
        return np.log(x)


def tanh(x):
    return np.tanh(x)


def sqrt(x):
    with np.errstate(all='ignore'):
        return np.sqrt(x)


def _float_unary(fn, x):
    """Float16(f(float(x))) for float16, f in the array's own precision otherwise (CX/numeric.h:59-83 over std::f).
    Pinned as a library routine (numpy / scipy follow the same libm definitions); tolerance-level parity only."""
    x = np.asarray(x)
    with np.errstate(all='ignore'):
        if x.dtype == np.float16:
            return fn(x.astype(np.float32)).astype(np.float16)
        return fn(x).astype(x.dtype)


def erf(x):
    from scipy import special
    return _float_unary(special.erf, x)


def expm1(x):
    return _float_unary(np.expm1, x)


def exp2(x):
    return _float_unary(np.exp2, x)


def log10(x):
    return _float_unary(np.log10, x)


def log2(x):
    return _float_unary(np.log2, x)


def log1p(x):
    return _float_unary(np.log1p, x)


def sinh(x):
    return _float_unary(np.sinh, x)


def cosh(x):
    return _float_unary(np.cosh, x)


def arcsinh(x):
    return _float_unary(np.arcsinh, x)


def arccosh(x):
    return _float_unary(np.arccosh, x)


def sin(x):
    return _float_unary(np.sin, x)


def cos(x):
    return _float_unary(np.cos, x)


def tan(x):
    return _float_unary(np.tan, x)


def arcsin(x):
    return _float_unary(np.arcsin, x)


def arccos(x):
    return _float_unary(np.arccos, x)


def arctan(x):
    return _float_unary(np.arctan, x)


def ceil(x):
    return _float_unary(np.ceil, x)


def floor(x):
    return _float_unary(np.floor, x)


def square(x):
    """SquareKernel: out = x * x in the array dtype, integers wrap (native/native_device/misc.cc)."""
    x = np.asarray(x)
    with np.errstate(all='ignore'):
        return (x * x).astype(x.dtype)


def absolute(x):
    """AbsKernel: std::abs, identity for uint8 (CX/numeric.h:40-57); abs(lowest) wraps to lowest."""
    x = np.asarray(x)
    with np.errstate(all='ignore'):
        return np.abs(x).astype(x.dtype)


def sign(x):
    """SignKernel: NaN passes, else (0 < x) - (x < 0) (CX/numeric.h:33-38)."""
    x = np.asarray(x)
    r = ((x > 0).astype(np.int8) - (x < 0).astype(np.int8)).astype(x.dtype)
    if x.dtype.kind == 'f':
        r = np.where(np.isnan(x), x, r).astype(x.dtype)
    return r


def logical_not(x):
    return ~np.asarray(x).astype(bool)


def isnan(x):
    x = np.asarray(x)
    return np.isnan(x) if x.dtype.kind == 'f' else np.zeros(x.shape, bool)


def isinf(x):
    x = np.asarray(x)
    return np.isinf(x) if x.dtype.kind == 'f' else np.zeros(x.shape, bool)


def isfinite(x):
    x = np.asarray(x)
    return np.isfinite(x) if x.dtype.kind == 'f' else np.ones(x.shape, bool)


def logical_and(x1, x2):
    return np.asarray(x1).astype(bool) & np.asarray(x2).astype(bool)


def logical_or(x1, x2):
    return np.asarray(x1).astype(bool) | np.asarray(x2).astype(bool)


def logical_xor(x1, x2):
    """!x1 != !x2 (native/native_device/logic.cc NativeLogicalXorKernel)."""
    return np.asarray(x1).astype(bool) ^ np.asarray(x2).astype(bool)


def power(x1, x2):
    """chainerx::Power (CX/numeric.h:85-135) on operands already cast to one dtype: integers by repeated squaring with
    wrap-around, a negative exponent gives +-1 for bases 1 / -1 and 0 otherwise; floats through pow."""
    x1, x2 = np.broadcast_arrays(np.asarray(x1), np.asarray(x2))
    dt = x1.dtype
    with np.errstate(all='ignore'):
        if dt.kind == 'f':
            if dt == np.float16:
                return np.power(x1.astype(np.float32), x2.astype(np.float32)).astype(np.float16)
            return np.power(x1, x2).astype(dt)
        out = np.ones(x1.shape, dt)
        base = x1.copy()
        e = np.where(x2 > 0, x2, 0).astype(np.uint64)
        while (e > 0).any():
            out = np.where((e & np.uint64(1)) != 0, out * base, out).astype(dt)
            base = (base * base).astype(dt)
            e = e >> np.uint64(1)
        if dt.kind == 'i':
            neg = x2 < 0
            odd = (x2 & 1) != 0
            special = np.where(x1 == 1, 1, np.where(x1 == -1, np.where(odd, -1, 1), 0)).astype(dt)
            out = np.where(neg, special, out).astype(dt)
        return out


def floor_divide(x1, x2):
    """native::FloorDivide (native/native_device/arithmetic.cc:107-139): integers floor towards -inf, 0 for a zero divisor;
    floats (x - fmod(x, y)) / y minus one when the remainder and the divisor disagree in sign; float16 through float."""
    x1, x2 = np.broadcast_arrays(np.asarray(x1), np.asarray(x2))
    dt = x1.dtype
    with np.errstate(all='ignore'):
        if dt.kind in 'iu':
            safe = np.where(x2 == 0, 1, x2).astype(dt)
            return np.where(x2 == 0, 0, np.floor_divide(x1, safe)).astype(dt)
        ct = np.float32 if dt == np.float16 else dt
        x, y = x1.astype(ct), x2.astype(ct)
        rem = np.fmod(x, y)
        fix = ((rem < 0) & (y > 0)) | ((rem > 0) & (y < 0))
        return (((x - rem) / y).astype(ct) - fix.astype(ct)).astype(dt)


def mod(x1, x2):
    """Mod (native/native_device/arithmetic.cc:260-295): result takes the divisor's sign; integers give 0 when either operand
    is 0, floats NaN for a zero divisor; float16 through float."""
    x1, x2 = np.broadcast_arrays(np.asarray(x1), np.asarray(x2))
    dt = x1.dtype
    with np.errstate(all='ignore'):
        if dt.kind in 'iu':
            safe = np.where(x2 == 0, 1, x2).astype(dt)
            return np.where((x1 == 0) | (x2 == 0), 0, np.mod(x1, safe)).astype(dt)
        ct = np.float32 if dt == np.float16 else dt
        x, y = x1.astype(ct), x2.astype(ct)
        r = np.fmod(x, y)
        fix = ((r > 0) & (y < 0)) | ((r < 0) & (y > 0))
        r = np.where(fix, (y + r).astype(ct), r)
        return np.where(y == 0, np.nan, r).astype(dt)


def bitwise_and(x1, x2):
    return np.bitwise_and(np.asarray(x1), np.asarray(x2))


def bitwise_or(x1, x2):
    return np.bitwise_or(np.asarray(x1), np.asarray(x2))


def bitwise_xor(x1, x2):
    return np.bitwise_xor(np.asarray(x1), np.asarray(x2))


def left_shift(x1, x2):
    """`x1 << x2` in the promoted type, narrowed back (counts within the type's width)."""
    x1, x2 = np.asarray(x1), np.asarray(x2)
    wide = np.left_shift(x1.astype(np.int64), x2.astype(np.int64))
    return wide.astype(x1.dtype)


def right_shift(x1, x2):
    x1, x2 = np.asarray(x1), np.asarray(x2)
    return np.right_shift(x1.astype(np.int64), x2.astype(np.int64)).astype(x1.dtype)


def fmod(x1, x2):
    """FmodKernel: std::fmod, float16 through float."""
    x1, x2 = np.asarray(x1), np.asarray(x2)
    with np.errstate(all='ignore'):
        if x1.dtype == np.float16:
            return np.fmod(x1.astype(np.float32), x2.astype(np.float32)).astype(np.float16)
        return np.fmod(x1, x2).astype(x1.dtype)


def arctan2(x1, x2):
    x1, x2 = np.asarray(x1), np.asarray(x2)
    with np.errstate(all='ignore'):
        if x1.dtype == np.float16:
            return np.arctan2(x1.astype(np.float32), x2.astype(np.float32)).astype(np.float16)
        return np.arctan2(x1, x2).astype(x1.dtype)


def where(condition, x, y, dtype):
    """WhereKernel family (native/native_device/indexing.cc:194-283): condition cast to bool, x / y cast to the out dtype."""
    c = np.asarray(condition).astype(bool)
    dt = np.dtype(dtype)
    xa = _scalar_as(x, dt) if np.isscalar(x) else np.asarray(x).astype(dt)
    ya = _scalar_as(y, dt) if np.isscalar(y) else np.asarray(y).astype(dt)
    return np.where(c, xa, ya).astype(dt)


def if_less_else(x1, x2, pos, neg):
    """x1 < x2 ? pos : neg (misc.cc:39-61); x2 and pos are scalars cast to the dtype."""
    x1 = np.asarray(x1)
    dt = np.asarray(neg).dtype
    return np.where(x1 < _scalar_as(x2, dt), _scalar_as(pos, dt), neg).astype(dt)


def relu(x):
    """Relu = Maximum(0, x) = IfLessElse(x, 0, 0, x) (CX/routines/activation.cc:80-84, misc.cc:210-216)."""
    return if_less_else(x, 0, 0, x)


def sigmoid(x):
    """Reciprocal(1 + Exp(-x)) as four kernels: MultiplyAS(-1), Exp, AddAS(1), DivideSA(1) (activation.cc:74-78)."""
    x = np.asarray(x)
    one = _scalar_as(1, x.dtype)
    with np.errstate(all='ignore'):
        neg = x * _scalar_as(-1, x.dtype)
        e = np.exp(neg)
        return one / (e + one)


def equal(x1, x2):
    return np.asarray(x1) == np.asarray(x2)


# ---------------------------------------------------------------------------------------------
# reductions (CX/native/reduce.h:46-83 order)
# ---------------------------------------------------------------------------------------------
def _rows(a, axes):
    """Moves the reduced axes last (kept in their own order: the native iterator walks the reduced axes in C order,
    CX/reduction_kernel_arg.cc:19-144) and flattens to [n_out, reduce_len]."""
    a = np.asarray(a)
    axes = tuple(sorted(ax % a.ndim for ax in axes))
    keep = [i for i in range(a.ndim) if i not in axes]
    t = a.transpose(keep + list(axes))
    out_shape = tuple(a.shape[i] for i in keep)
    red = int(np.prod([a.shape[i] for i in axes], dtype=np.int64)) if axes else 1
    return np.ascontiguousarray(t).reshape(-1, red), out_shape, axes


def _axes_of(a, axis):
    if axis is None:
        return tuple(range(np.asarray(a).ndim))
    if isinstance(axis, (int, np.integer)):
        return (int(axis),)
    return tuple(axis)


def _restore(out, out_shape, a, axes, keepdims):
    out = out.reshape(out_shape)
    if keepdims:
        shape = [1 if i in axes else d for i, d in enumerate(np.asarray(a).shape)]
        out = out.reshape(shape)
    return out


def sum(a, axis=None, keepdims=False):
    """NativeSumKernel (reduction.cc:96-119): int/bool inputs accumulate in int64 (CX/routines/reduction.cc:34-49),
    float16 accumulates in float32 and rounds once, float32/64 accumulate in their own type, pairwise order.
    parity unpinned (bit level) for float data: the order is derived from the source; integer-valued data pins it exactly."""
    a = np.asarray(a)
    rows, out_shape, axes = _rows(a, _axes_of(a, axis))
    n, length = rows.shape
    L = lib()
    if a.dtype.kind in 'biu':
        r = _c(rows, np.int64)
        out = np.empty(n, np.int64)
        L.oracle_sum_i64(_ptr(r, _i64p), _i64(n), _i64(length), _ptr(out, _i64p))
    elif a.dtype == np.float32:
        out = np.empty(n, np.float32)
        L.oracle_sum_f32(_ptr(rows, _f32p), _i64(n), _i64(length), _ptr(out, _f32p))
    elif a.dtype == np.float64:
        out = np.empty(n, np.float64)
        L.oracle_sum_f64(_ptr(rows, _f64p), _i64(n), _i64(length), _ptr(out, _f64p))
    elif a.dtype == np.float16:
        bits = rows.view(np.uint16)
        ob = np.empty(n, np.uint16)
        L.oracle_sum_f16(_ptr(bits, _u16p), _i64(n), _i64(length), _ptr(ob, _u16p))
        out = ob.view(np.float16)
    else:
        raise TypeError(a.dtype)
    return _restore(out, out_shape, a, axes, keepdims)


def amax(a, axis=None, keepdims=False):
    """NativeAMaxKernel (statistics.cc:27-48): NaN-propagating maximum, identity lowest / -inf."""
    a = np.asarray(a)
    rows, out_shape, axes = _rows(a, _axes_of(a, axis))
    n, length = rows.shape
    L = lib()
    if a.dtype.kind == 'f' and a.dtype != np.float64:
        r = _c(rows, np.float32)  # float16 -> float32 is exact and order preserving
        out = np.empty(n, np.float32)
        L.oracle_amax_f32(_ptr(r, _f32p), _i64(n), _i64(length), _ptr(out, _f32p))
        out = out.astype(a.dtype)
    elif a.dtype == np.float64:
        out = np.empty(n, np.float64)
        L.oracle_amax_f64(_ptr(rows, _f64p), _i64(n), _i64(length), _ptr(out, _f64p))
    else:
        r = _c(rows, np.int64)
        lowest = 0 if a.dtype.kind in 'bu' else int(np.iinfo(a.dtype).min)
        out = np.empty(n, np.int64)
        L.oracle_amax_i64(_ptr(r, _i64p), _i64(n), _i64(length), _i64(lowest), _ptr(out, _i64p))
        out = out.astype(a.dtype)
    return _restore(out, out_shape, a, axes, keepdims)


def argmax(a, axis=None):
    """NativeArgMaxKernel (reduction.cc:34-61) through the pairwise tree: the earlier index wins a tie inside a
    32-element block (and in the tail), the later block wins a tie between blocks; NaN never replaces and a leading
    NaN is never replaced.  The index counts positions in the C-order flattening of the reduced axes."""
    a = np.asarray(a)
    rows, out_shape, axes = _rows(a, _axes_of(a, axis))
    n, length = rows.shape
    r = _c(rows, np.float64)
    out = np.empty(n, np.int64)
    lib().oracle_argmax(_ptr(r, _f64p), _i64(n), _i64(length), _ptr(out, _i64p))
    return out.reshape(out_shape)


def amin(a, axis=None, keepdims=False):
    """NativeAMinKernel (statistics.cc:52-73) is AMax with the comparison mirrored: through an order-reversing exact map
    (negation for floats, bitwise complement for integers) the same pairwise tree and NaN rule apply."""
    a = np.asarray(a)
    if a.dtype.kind == 'f':
        return -amax(-a, axis, keepdims)
    if a.dtype.kind == 'b':
        return ~amax(~a, axis, keepdims)
    wide = ~a.astype(np.int64)
    return (~amax(wide, axis, keepdims)).astype(a.dtype)


def argmin(a, axis=None):
    """NativeArgMinKernel (reduction.cc:65-92): ArgMax's accumulator with `accum.min > next.min`."""
    a = np.asarray(a)
    if a.dtype.kind == 'f':
        return argmax(-a.astype(np.float64), axis)
    return argmax(-(a.astype(np.float64)), axis)


def nanargmax(a, axis=None):
    """NanArgMax routine (CX/routines/sorting.cc:93-126): NaN -> -inf, then ArgMax."""
    a = np.asarray(a)
    return argmax(np.where(np.isnan(a), -np.inf, a).astype(a.dtype) if a.dtype.kind == 'f' else a, axis)


def nanargmin(a, axis=None):
    a = np.asarray(a)
    return argmin(np.where(np.isnan(a), np.inf, a).astype(a.dtype) if a.dtype.kind == 'f' else a, axis)


def all(a, axis=None, keepdims=False):
    """NativeAllKernel (logic.cc): input cast to bool, accum && next; order independent."""
    a = np.asarray(a).astype(bool)
    return np.all(a, axis=axis if axis is None or isinstance(axis, int) else tuple(axis), keepdims=keepdims)


def any(a, axis=None, keepdims=False):
    """NativeAnyKernel (logic.cc): input cast to bool, accum || next; order independent."""
    a = np.asarray(a).astype(bool)
    return np.any(a, axis=axis if axis is None or isinstance(axis, int) else tuple(axis), keepdims=keepdims)


def cumsum(a, axis=None):
    """NativeCumsumKernel (reduction.cc:121-144) over native::Scan (reduce.h:98-113): strictly serial prefix sums in the
    accumulator type (float for float16 with every prefix rounded on output, int64 for bool / integer inputs)."""
    a = np.asarray(a)
    if axis is None:
        a = a.reshape(-1)
        axis = 0
    if a.dtype.kind in 'biu':
        return np.cumsum(a.astype(np.int64), axis=axis)
    acc_t = np.float32 if a.dtype == np.float16 else a.dtype
    moved = np.moveaxis(a, axis, -1)
    out = np.empty(moved.shape, a.dtype)
    acc = np.zeros(moved.shape[:-1], acc_t)
    with np.errstate(all='ignore'):
        for j in range(moved.shape[-1]):
            acc = (acc + moved[..., j].astype(acc_t)).astype(acc_t)
            out[..., j] = acc.astype(a.dtype)
    return np.moveaxis(out, -1, axis)


def nansum(a, axis=None, keepdims=False):
    """Nansum routine (CX/routines/reduction.cc:149-170): NaNs replaced by 0, then the Sum kernel."""
    a = np.asarray(a)
    if a.dtype.kind == 'f':
        a = np.where(np.isnan(a), a.dtype.type(0), a)
    return sum(a, axis, keepdims)


def add_at(a, indices, axis, b, mode=None):
    """NativeAddAtKernel (indexing.cc:107-190): copy of a, then for every index in C order out[.., index, ..] += b[.., i, ..]
    in the array dtype (float16 rounds after every addition, integers wrap, bool saturates to True)."""
    a, indices, b = np.asarray(a), np.asarray(indices), np.asarray(b)
    axis = axis % a.ndim
    dim = a.shape[axis]
    out = np.moveaxis(a.copy(), axis, 0)
    nleft = axis
    bm = np.moveaxis(b.reshape(a.shape[:axis] + (-1,) + a.shape[axis + 1:]), nleft, 0)
    with np.errstate(all='ignore'):
        for i, index in enumerate(indices.reshape(-1).tolist()):
            if mode in (None, 'raise'):
                if index < -dim or index >= dim:
                    raise IndexError('Index %d is out of bounds for axis %d with size %d' % (index, axis, dim))
                if index < 0:
                    index += dim
            elif mode == 'wrap':
                index = dim - ((-index + dim - 1) % dim + 1) if index < 0 else index % dim
            else:
                index = max(0, min(index, dim - 1))
            if a.dtype == np.bool_:
                out[index] = out[index] | bm[i]
            elif a.dtype == np.float16:
                out[index] = (out[index].astype(np.float32) + bm[i].astype(np.float32)).astype(np.float16)
            else:
                out[index] = (out[index] + bm[i]).astype(a.dtype)
    return np.moveaxis(out, 0, axis)


def identity(n, dtype):
    return np.identity(n, dtype)


def eye(n, m, k, dtype):
    return np.eye(n, m, k, dtype)


def tri(n, m, k, dtype):
    return np.tri(n, m, k, dtype)


def linspace(start, stop, num, endpoint, dtype):
    """NativeLinspaceKernel (fill.cc): (start*(n-1-i) + stop*i)/(n-1) in double, cast to the dtype."""
    start, stop = float(start), float(stop)
    if not endpoint:
        stop = start + (stop - start) * (num - 1) / num
    i = np.arange(num, dtype=np.float64)
    v = np.full(num, start) if num == 1 else (start * (num - 1 - i) + stop * i) / (num - 1)
    with np.errstate(all='ignore'):
        return v.astype(dtype)


def diagflat(v, k):
    return np.diagflat(np.asarray(v), k)


def mean(a, axis=None, keepdims=False):
    """Mean = SumKernel into the float result dtype, then DivideASKernel by the count (CX/routines/statistics.cc:95-154)."""
    a = np.asarray(a)
    dt = a.dtype if a.dtype.kind == 'f' else np.dtype(np.float32)
    axes = _axes_of(a, axis)
    n = int(np.prod([a.shape[i] for i in axes], dtype=np.int64))
    s = sum(a.astype(dt), axis, keepdims)
    return (s / _scalar_as(n, dt)).astype(dt)


def logsumexp(x, axis=None, keepdims=False):
    """CX/routines/reduction.cc:78-86."""
    x = np.asarray(x)
    axes = _axes_of(x, axis)
    xmax = amax(x, axes, True)
    logs = log(sum(exp(subtract(x, xmax)), axes, keepdims))
    return add(xmax if keepdims else xmax.reshape(logs.shape), logs)


def log_softmax(x, axis=None):
    """x - LogSumExp(x, axis or 1, keepdims=True) (CX/routines/reduction.cc:88-92)."""
    x = np.asarray(x)
    return subtract(x, logsumexp(x, 1 if axis is None else axis, True))


# ---------------------------------------------------------------------------------------------
# dot / linear / conv
# ---------------------------------------------------------------------------------------------
def dot(a, b):
    """NativeDotKernel without BLAS (dot.cc:181-227).  parity unpinned (bit level): exact fp32 bit patterns follow the
    (i, l, j) fmaf order read from the source; the reference's literal vectors and integer-valued matrices pin the rest."""
    a, b = np.asarray(a), np.asarray(b)
    assert a.ndim == 2 and b.ndim == 2 and a.shape[1] == b.shape[0] and a.dtype == b.dtype
    m, k = a.shape
    n = b.shape[1]
    L = lib()
    ac, bc = _c(a), _c(b)
    if a.dtype == np.float32:
        out = np.empty((m, n), np.float32)
        L.oracle_dot_f32(_ptr(ac, _f32p), _ptr(bc, _f32p), _ptr(out, _f32p), _i64(m), _i64(k), _i64(n))
    elif a.dtype == np.float64:
        out = np.empty((m, n), np.float64)
        L.oracle_dot_f64(_ptr(ac, _f64p), _ptr(bc, _f64p), _ptr(out, _f64p), _i64(m), _i64(k), _i64(n))
    elif a.dtype == np.float16:
        ob = np.empty((m, n), np.uint16)
        rc = L.oracle_dot_f16(_ptr(ac.view(np.uint16), _u16p), _ptr(bc.view(np.uint16), _u16p), _ptr(ob, _u16p), _i64(m), _i64(k), _i64(n))
        assert rc == 0
        out = ob.view(np.float16)
    elif a.dtype == np.bool_:
        # MultiplyAdd(bool, bool, bool) = (x && y) || z (dot.cc:134)
        out = (ac.astype(np.int64) @ bc.astype(np.int64)) != 0
    elif a.dtype.kind in 'iu':
        # one accumulator of the array dtype per element, acc = a*b + acc (dot.cc:130-132, 200-214): the sum modulo 2^bits,
        # whatever the order; computed modulo 2^64 (numpy's integer matmul wraps) and truncated
        with np.errstate(over='ignore'):
            out = (ac.astype(np.uint64) @ bc.astype(np.uint64)).astype(a.dtype)
    else:
        raise TypeError(a.dtype)
    return out


def linear(x, w, b=None):
    """Linear (CX/routines/connection.cc:322-394): Dot(x, w.T) then AddKernel with the broadcast bias."""
    x, w = np.asarray(x), np.asarray(w)
    x2 = x.reshape(x.shape[0], -1)
    y = dot(x2, np.ascontiguousarray(w.T))
    if b is not None:
        y = add(y, np.broadcast_to(b, y.shape))
    return y


def conv_out_dim(in_dim, k, s, p, cover_all):
    """GetConvOutDim (CX/routines/connection.cc:37-49)."""
    num = in_dim + 2 * p - k + (s - 1 if cover_all else 0)
    if num < 0:
        raise ValueError('Output size should be positive.')
    return num // s + 1


def _pair(v):
    return (int(v), int(v)) if isinstance(v, (int, np.integer)) else (int(v[0]), int(v[1]))


def conv(x, w, b=None, stride=1, pad=0, cover_all=False):
    """NativeConvKernel (conv.cc:41-89); returns contiguous NCHW values."""
    x, w = np.asarray(x), np.asarray(w)
    assert x.dtype == w.dtype
    N, C, H, W = x.shape
    K, C2, R, S = w.shape
    assert C == C2
    sh, sw = _pair(stride)
    ph, pw = _pair(pad)
    OH = conv_out_dim(H, R, sh, ph, cover_all)
    OW = conv_out_dim(W, S, sw, pw, cover_all)
    L = lib()
    xc, wc = _c(x), _c(w)
    bc = _c(b, x.dtype) if b is not None else None
    args = [_i64(v) for v in (N, C, H, W, K, R, S, sh, sw, ph, pw, OH, OW)]
    if x.dtype == np.float32:
        out = np.empty((N, K, OH, OW), np.float32)
        rc = L.oracle_conv_f32(_ptr(xc, _f32p), _ptr(wc, _f32p), _ptr(bc, _f32p) if bc is not None else None, _ptr(out, _f32p), *args)
    elif x.dtype == np.float64:
        out = np.empty((N, K, OH, OW), np.float64)
        rc = L.oracle_conv_f64(_ptr(xc, _f64p), _ptr(wc, _f64p), _ptr(bc, _f64p) if bc is not None else None, _ptr(out, _f64p), *args)
    elif x.dtype == np.float16:
        ob = np.empty((N, K, OH, OW), np.uint16)
        rc = L.oracle_conv_f16(_ptr(xc.view(np.uint16), _u16p), _ptr(wc.view(np.uint16), _u16p),
                               _ptr(bc.view(np.uint16), _u16p) if bc is not None else None, _ptr(ob, _u16p), *args)
        out = ob.view(np.float16)
    else:
        raise TypeError(x.dtype)
    assert rc == 0
    return out


# ---------------------------------------------------------------------------------------------
# normalization / pooling / indexing
# ---------------------------------------------------------------------------------------------
def fixed_batch_norm(x, gamma, beta, mean, var, eps=2e-5, axis=None):
    """GenericFixedBatchNormKernel (CX/routines/normalization.cc:251-264 -> ApplyGenericBatchNorm :113-153):
    interm dtype = promotion of the five operands; inv_std = 1 / sqrt(var + eps);
    out = ((x - mean) * inv_std) * gamma + beta, one rounding per operation in the interm dtype, cast back to x's."""
    x = np.asarray(x)
    axes = (0,) if axis is None else tuple(sorted(_axes_of(x, axis)))
    red_shape = tuple(1 if i in axes else d for i, d in enumerate(x.shape))
    dt = np.result_type(x.dtype, *[np.asarray(p).dtype for p in (gamma, beta, mean, var)])
    g, b, m, v = [np.asarray(p).reshape(red_shape).astype(dt) for p in (gamma, beta, mean, var)]
    xc = x.astype(dt)
    with np.errstate(all='ignore'):
        inv_std = _scalar_as(1, dt) / np.sqrt(v + _scalar_as(eps, dt))
        out = (xc - m) * inv_std * g + b
    return out.astype(x.dtype)


def _tuple_n(v, n):
    if isinstance(v, (int, np.integer)):
        return (int(v),) * n
    v = tuple(int(i) for i in v)
    assert len(v) == n, (v, n)
    return v


def _windows_nd(x, ksize, stride, pad, cover_all, pad_value):
    """Im2Col over n spatial axes (CX/native/im2col.cc:82-149): [N, C, k_1..k_n, o_1..o_n]; the padded copy of x is filled with
    `pad_value` (cover_all adds stride - 1 more on the high side) and one strided view per kernel offset is copied out."""
    n = x.ndim - 2
    out_dims = tuple(conv_out_dim(x.shape[2 + d], ksize[d], stride[d], pad[d], cover_all) for d in range(n))
    padded_shape = x.shape[:2] + tuple(x.shape[2 + d] + 2 * pad[d] + (stride[d] - 1 if cover_all else 0) for d in range(n))
    padded = np.full(padded_shape, pad_value, x.dtype)
    padded[(slice(None), slice(None)) + tuple(slice(pad[d], pad[d] + x.shape[2 + d]) for d in range(n))] = x
    col = np.empty(x.shape[:2] + tuple(ksize) + out_dims, x.dtype)
    for kidx in np.ndindex(*ksize):
        src = (slice(None), slice(None)) + tuple(slice(kidx[d], kidx[d] + stride[d] * out_dims[d], stride[d]) for d in range(n))
        col[(slice(None), slice(None)) + kidx] = padded[src]
    return col


def conv_nd(x, w, b=None, stride=1, pad=0, cover_all=False):
    """NativeConvKernel for any number of spatial axes (conv.cc:41-89): Im2Col, TensorDot(col, w) over (channel, k_1..k_n) --
    native Dot, float16 accumulating in float -- then `y += b` in the array dtype, then the channel axis moved to position 1."""
    x, w = np.asarray(x), np.asarray(w)
    assert x.dtype == w.dtype and x.ndim == w.ndim and x.shape[1] == w.shape[1]
    n = x.ndim - 2
    stride, pad = _tuple_n(stride, n), _tuple_n(pad, n)
    col = _windows_nd(x, w.shape[2:], stride, pad, cover_all, 0)
    axes = tuple(range(1, n + 2))
    y = _tensordot(col, w, axes, axes)  # [N, o_1..o_n, K]
    if b is not None:
        y = add(y, np.broadcast_to(np.asarray(b).astype(y.dtype), y.shape))
    return np.ascontiguousarray(np.moveaxis(y, -1, 1))


def max_pool_nd(x, ksize, stride=None, pad=0, cover_all=False):
    """NativeMaxPoolKernel over n spatial axes (pool.cc:69-94): Im2Col padded with the lowest value, AMax over the kernel axes."""
    x = np.asarray(x)
    n = x.ndim - 2
    ksize = _tuple_n(ksize, n)
    stride = ksize if stride is None else _tuple_n(stride, n)
    col = _windows_nd(x, ksize, stride, _tuple_n(pad, n), cover_all, _lowest(x.dtype))
    return amax(col, tuple(range(2, 2 + n)))


def average_pool_nd(x, ksize, stride=None, pad=0, pad_mode='ignore'):
    """NativeAveragePoolKernel over n spatial axes (pool.cc:191-302): zero-padded Im2Col, Sum over the kernel axes (an array of the
    input dtype), divided by the window size ('zero') or by the number of window positions inside the array ('ignore'): the outer
    product of the per-axis widths, built in the array dtype."""
    x = np.asarray(x)
    n = x.ndim - 2
    ksize = _tuple_n(ksize, n)
    stride = ksize if stride is None else _tuple_n(stride, n)
    pad = _tuple_n(pad, n)
    col = _windows_nd(x, ksize, stride, pad, False, 0)
    s = sum(col, tuple(range(2, 2 + n)))
    if pad_mode == 'zero':
        with np.errstate(all='ignore'):
            return (s / _scalar_as(int(np.prod(ksize)), x.dtype)).astype(x.dtype)
    widths = None
    for i in range(n):
        d, k, st, p = x.shape[2 + i], ksize[i], stride[i], pad[i]
        n_out = conv_out_dim(d, k, st, p, False)
        start = np.arange(n_out).astype(x.dtype) * _scalar_as(st, x.dtype) - _scalar_as(p, x.dtype)
        end = start + _scalar_as(k, x.dtype)
        w = (np.minimum(end, _scalar_as(d, x.dtype)) - np.maximum(start, _scalar_as(0, x.dtype))).astype(x.dtype)
        widths = w if widths is None else (widths[..., None] * w).astype(x.dtype)
    with np.errstate(all='ignore'):
        return (s / widths).astype(x.dtype)


def _windows(x, ksize, stride, pad, cover_all, pad_value):
    """Im2Col (CX/native/im2col.cc:82-149): [N,C,kh,kw,OH,OW] with `pad_value` outside the image."""
    N, C, H, W = x.shape
    kh, kw = ksize
    sh, sw = stride
    ph, pw = pad
    OH = conv_out_dim(H, kh, sh, ph, cover_all)
    OW = conv_out_dim(W, kw, sw, pw, cover_all)
    eh = sh - 1 if cover_all else 0
    ew = sw - 1 if cover_all else 0
    padded = np.full((N, C, H + 2 * ph + eh, W + 2 * pw + ew), pad_value, x.dtype)
    padded[:, :, ph:ph + H, pw:pw + W] = x
    col = np.empty((N, C, kh, kw, OH, OW), x.dtype)
    for r in range(kh):
        for s in range(kw):
            col[:, :, r, s] = padded[:, :, r:r + sh * OH:sh, s:s + sw * OW:sw]
    return col


def _lowest(dtype):
    dtype = np.dtype(dtype)
    if dtype.kind == 'f':
        return -np.inf
    if dtype.kind == 'b':
        return False
    return np.iinfo(dtype).min


def max_pool(x, ksize, stride=None, pad=0, cover_all=False):
    """NativeMaxPoolKernel (pool.cc:69-94): Im2Col padded with lowest/-inf, then AMax over the window axes."""
    x = np.asarray(x)
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    col = _windows(x, ksize, stride, _pair(pad), cover_all, _lowest(x.dtype))
    return amax(col, (2, 3))


def average_pool(x, ksize, stride=None, pad=0, pad_mode='ignore'):
    """NativeAveragePoolKernel (pool.cc:252-302): zero-padded Im2Col, SumKernel over the window, then DivideAS by the
    window size ('zero') or Divide by the per-position count of in-image taps ('ignore', :197-250)."""
    x = np.asarray(x)
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    col = _windows(x, ksize, stride, pad, False, 0)
    s = sum(col, (2, 3))
    if pad_mode == 'zero':
        with np.errstate(all='ignore'):
            return (s / _scalar_as(ksize[0] * ksize[1], x.dtype)).astype(x.dtype)
    widths = None
    for i in range(2):
        d, k, st, p = x.shape[2 + i], ksize[i], stride[i], pad[i]
        n_out = conv_out_dim(d, k, st, p, False)
        start = np.arange(n_out).astype(x.dtype) * _scalar_as(st, x.dtype) - _scalar_as(p, x.dtype)
        end = start + _scalar_as(k, x.dtype)
        w = (np.minimum(end, _scalar_as(d, x.dtype)) - np.maximum(start, _scalar_as(0, x.dtype))).astype(x.dtype)
        widths = w if widths is None else (widths[:, None] * w[None, :]).astype(x.dtype)
    with np.errstate(all='ignore'):
        return (s / widths).astype(x.dtype)


def _col2im(col, stride, pad, out_size):
    """native_internal::Col2Im (CX/native/col2im.cc:22-122): zero array of the padded size, `+=` per kernel offset in (r, s)
    order, every addition rounded to the array dtype (float16 through float), padding cut off."""
    n, c, kh, kw, h, w = col.shape
    sh, sw = stride
    ph, pw = pad
    oh, ow = out_size
    padded = np.zeros((n, c, oh + 2 * ph + sh - 1, ow + 2 * pw + sw - 1), col.dtype)
    with np.errstate(all='ignore'):
        for r in range(kh):
            for q in range(kw):
                view = padded[:, :, r:r + sh * h:sh, q:q + sw * w:sw]
                view[...] = add(view, col[:, :, r, q])
    return padded[:, :, ph:ph + oh, pw:pw + ow]


def _tensordot(a, b, a_axes, b_axes):
    """TensorDot (CX/native/tensor_dot.cc:63-99): roll, reshape to 2-D, native Dot."""
    a, b = np.asarray(a), np.asarray(b)
    a_keep = [i for i in range(a.ndim) if i not in a_axes]
    b_keep = [i for i in range(b.ndim) if i not in b_axes]
    red = int(np.prod([a.shape[i] for i in a_axes], dtype=np.int64))
    a2 = a.transpose(a_keep + list(a_axes)).reshape(-1, red)
    b2 = b.transpose(list(b_axes) + b_keep).reshape(red, -1)
    return dot(a2, b2).reshape(tuple(a.shape[i] for i in a_keep) + tuple(b.shape[i] for i in b_keep))


def conv_grad_weight(w_shape, x, gy, stride=1, pad=0, cover_all=False):
    """NativeConvGradWeightKernel (conv.cc:91-124): Im2Col(x) then TensorDot(gy, col) over batch and output positions."""
    x, gy = np.asarray(x), np.asarray(gy)
    col = _windows(x, tuple(w_shape[2:]), _pair(stride), _pair(pad), cover_all, 0)
    return _tensordot(gy, col, (0, 2, 3), (0, 4, 5))


def conv_transpose(x, w, b=None, stride=1, pad=0, out_size=None):
    """NativeConvTransposeKernel (conv.cc:126-160): TensorDot(w, x) over the input channels, batch axis first, Col2Im, bias."""
    x, w = np.asarray(x), np.asarray(w)
    stride, pad = _pair(stride), _pair(pad)
    kh, kw = w.shape[2:]
    if out_size is None:
        out_size = tuple(st * (d - 1) + k - 2 * p for d, k, st, p in zip(x.shape[2:], (kh, kw), stride, pad))
    col = _tensordot(w, x, (0,), (1,)).transpose(3, 0, 1, 2, 4, 5)
    out = np.ascontiguousarray(_col2im(np.ascontiguousarray(col), stride, pad, _pair(out_size)))
    if b is not None:
        out = add(out, np.broadcast_to(np.asarray(b).reshape(1, -1, 1, 1), out.shape))
    return out


def var(a, axis=None, keepdims=False):
    """Var (CX/routines/statistics.cc:147-154)."""
    a = np.asarray(a)
    axes = _axes_of(a, axis)
    diff = subtract(a, np.broadcast_to(mean(a, axes, True), a.shape))
    return mean(multiply(diff, diff), axes, keepdims)


def batch_norm(x, gamma, beta, running_mean, running_var, eps=2e-5, decay=0.9, axis=None):
    """GenericBatchNormKernel (CX/routines/normalization.cc:155-193).  Returns (out, new_running_mean, new_running_var,
    (x_mean, x_inv_std)).  The statistics and the normalisation run in ResultType(x, gamma, beta) (:176-180) -- float32 for a
    float16 x with float32 parameters -- and out is cast back to x's dtype (:143); the state keeps the promoted dtype."""
    x_in = np.asarray(x)
    dt = np.result_type(x_in.dtype, np.asarray(gamma).dtype, np.asarray(beta).dtype)
    x = x_in.astype(dt, copy=False)
    gamma, beta = np.asarray(gamma).astype(dt, copy=False), np.asarray(beta).astype(dt, copy=False)
    axes = tuple(sorted(a % x.ndim for a in ((0,) + tuple(range(2, x.ndim)) if axis is None else axis)))
    red = tuple(1 if i in axes else d for i, d in enumerate(x.shape))
    x_mean = mean(x, axes, True)
    x_var = var(x, axes, True)
    g, bt = np.asarray(gamma).reshape(red), np.asarray(beta).reshape(red)
    B = lambda v: np.broadcast_to(v, x.shape)
    inv_std = divide(_scalar_as(1, dt), sqrt(add(x_var, _scalar_as(eps, dt))))
    out = add(multiply(multiply(subtract(x, B(x_mean)), B(inv_std)), B(g)), B(bt))
    n = x.size // max(1, np.asarray(gamma).size)
    inv_decay = 1.0 - float(decay)
    rdt = np.asarray(running_mean).dtype  # running *= decay; running += (...).AsType(running dtype) (:185-190)
    rm = add(multiply(np.asarray(running_mean).reshape(red), _scalar_as(decay, rdt)), multiply(x_mean, _scalar_as(inv_decay, dt)).astype(rdt, copy=False))
    rv = add(multiply(np.asarray(running_var).reshape(red), _scalar_as(decay, rdt)),
             multiply(x_var, _scalar_as(inv_decay * (float(n) / max(n - 1, 1)), dt)).astype(rdt, copy=False))
    shp = np.asarray(gamma).shape
    return out.astype(x_in.dtype, copy=False), rm.reshape(shp), rv.reshape(shp), (x_mean, inv_std)


def batch_norm_grad(x, gamma, gout, state, axis=None):
    """GenericBatchNormGradKernel (CX/routines/normalization.cc:195-250): (gx, ggamma, gbeta).  Computed in the state's dtype
    (:224-232); gx is cast to x's dtype, ggamma to gamma's, gbeta to the state's beta dtype -- taken to be gamma's here (:234-246)."""
    x_in, gout = np.asarray(x), np.asarray(gout)
    x_mean, x_inv_std = state
    dt = np.asarray(x_mean).dtype
    x, gout = x_in.astype(dt, copy=False), gout.astype(dt, copy=False)
    gamma_dtype = np.asarray(gamma).dtype
    gamma = np.asarray(gamma).astype(dt, copy=False)
    axes = tuple(sorted(a % x.ndim for a in ((0,) + tuple(range(2, x.ndim)) if axis is None else axis)))
    red = tuple(1 if i in axes else d for i, d in enumerate(x.shape))
    B = lambda v: np.broadcast_to(v, x.shape)
    n = x.size // max(1, np.asarray(gamma).size)
    x_hat = multiply(subtract(x, B(x_mean)), B(x_inv_std))
    ggamma = sum(multiply(gout, x_hat), axes, True)
    gbeta = sum(gout, axes, True)
    g = np.asarray(gamma).reshape(red)
    inner = multiply(add(multiply(x_hat, B(ggamma)), B(gbeta)), _scalar_as(1.0 / n, dt))
    gx = multiply(B(multiply(g, x_inv_std)), subtract(gout, inner))
    shp = np.asarray(gamma).shape
    return gx.astype(x_in.dtype, copy=False), ggamma.reshape(shp).astype(gamma_dtype, copy=False), gbeta.reshape(shp).astype(gamma_dtype, copy=False)


def max_pool_grad(x, gout, ksize, stride=None, pad=0, cover_all=False):
    """NativeMaxPoolGradKernel (pool.cc:97-143): ArgMax of the -inf padded windows (native tie rule), gout added at that
    kernel offset of a zero col, Col2Im."""
    x, gout = np.asarray(x), np.asarray(gout)
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    col = _windows(x, ksize, stride, pad, cover_all, _lowest(x.dtype))
    idx = argmax(col, (2, 3))
    taps = np.arange(ksize[0] * ksize[1]).reshape(1, 1, ksize[0], ksize[1], 1, 1)
    gcol = np.where(idx[:, :, None, None] == taps, gout[:, :, None, None], np.zeros((), x.dtype)).astype(x.dtype)
    return np.ascontiguousarray(_col2im(gcol, stride, pad, x.shape[2:]))


def max_pool_grad_grad(x, ggx, ksize, stride=None, pad=0, cover_all=False):
    """NativeMaxPoolGradGradKernel (pool.cc:147-177): ggx's window element at the ArgMax position of x's window."""
    x, ggx = np.asarray(x), np.asarray(ggx)
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    idx = argmax(_windows(x, ksize, stride, pad, cover_all, _lowest(x.dtype)), (2, 3))
    col = _windows(ggx, ksize, stride, pad, cover_all, _lowest(x.dtype)).transpose(0, 1, 4, 5, 2, 3)
    flat = col.reshape(col.shape[:4] + (-1,))
    return np.take_along_axis(flat, idx[..., None], axis=-1)[..., 0]


def average_pool_grad(x, gout, ksize, stride=None, pad=0, pad_mode='ignore'):
    """NativeAveragePoolGradKernel (pool.cc:304-346)."""
    x, gout = np.asarray(x), np.asarray(gout)
    ksize = _pair(ksize)
    stride = ksize if stride is None else _pair(stride)
    pad = _pair(pad)
    n, c, oh, ow = gout.shape
    g = gout
    if pad_mode == 'ignore':
        widths = None
        for i in range(2):
            d, k, st, p = x.shape[2 + i], ksize[i], stride[i], pad[i]
            start = np.arange(gout.shape[2 + i]).astype(x.dtype) * _scalar_as(st, x.dtype) - _scalar_as(p, x.dtype)
            end = start + _scalar_as(k, x.dtype)
            w = (np.minimum(end, _scalar_as(d, x.dtype)) - np.maximum(start, _scalar_as(0, x.dtype))).astype(x.dtype)
            widths = w if widths is None else (widths[:, None] * w[None, :]).astype(x.dtype)
        g = divide(gout, np.broadcast_to(widths, gout.shape))
    gcol = np.broadcast_to(g[:, :, None, None], (n, c, ksize[0], ksize[1], oh, ow))
    gx = np.ascontiguousarray(_col2im(gcol, stride, pad, x.shape[2:]))
    if pad_mode == 'zero':
        gx = divide(gx, _scalar_as(ksize[0] * ksize[1], x.dtype))
    return gx


def _col2im_nd(col, stride, pad, out_size):
    """native_internal::Col2Im over n spatial axes (CX/native/col2im.cc:22-122): col [N, C, k_1..k_n, o_1..o_n]; a zero array of the
    padded size (stride - 1 more on the high side) receives one strided in-place `+=` per kernel offset in C order, every addition
    rounded to the array dtype; the padding is cut off."""
    n = len(out_size)
    ksize, odims = col.shape[2:2 + n], col.shape[2 + n:]
    padded = np.zeros(col.shape[:2] + tuple(out_size[d] + 2 * pad[d] + stride[d] - 1 for d in range(n)), col.dtype)
    with np.errstate(all='ignore'):
        for kidx in np.ndindex(*ksize):
            sel = (slice(None), slice(None)) + tuple(slice(kidx[d], kidx[d] + stride[d] * odims[d], stride[d]) for d in range(n))
            view = padded[sel]
            view[...] = add(view, col[(slice(None), slice(None)) + kidx])
    return padded[(slice(None), slice(None)) + tuple(slice(pad[d], pad[d] + out_size[d]) for d in range(n))]


def conv_grad_weight_nd(w_shape, x, gy, stride=1, pad=0, cover_all=False):
    """NativeConvGradWeightKernel for any number of spatial axes (conv.cc:91-124): Im2Col(x), TensorDot(gy, col) over the batch axis
    and the output positions."""
    x, gy = np.asarray(x), np.asarray(gy)
    n = x.ndim - 2
    col = _windows_nd(x, tuple(w_shape[2:]), _tuple_n(stride, n), _tuple_n(pad, n), cover_all, 0)
    out_axes = tuple(range(2, 2 + n))
    return _tensordot(gy, col, (0,) + out_axes, (0,) + tuple(a + n for a in out_axes))


def conv_transpose_nd(x, w, b=None, stride=1, pad=0, out_size=None):
    """NativeConvTransposeKernel for any number of spatial axes (conv.cc:126-160): TensorDot(w, x) over the input channels gives
    [C_out, k_1..k_n, N, i_1..i_n], the batch axis is moved first, Col2Im, then the bias."""
    x, w = np.asarray(x), np.asarray(w)
    n = x.ndim - 2
    stride, pad = _tuple_n(stride, n), _tuple_n(pad, n)
    ksize = w.shape[2:]
    if out_size is None:
        out_size = tuple(st * (d - 1) + k - 2 * p for d, k, st, p in zip(x.shape[2:], ksize, stride, pad))
    col = np.moveaxis(_tensordot(w, x, (0,), (1,)), n + 1, 0)
    out = np.ascontiguousarray(_col2im_nd(np.ascontiguousarray(col), stride, pad, _tuple_n(out_size, n)))
    if b is not None:
        out = add(out, np.broadcast_to(np.asarray(b).reshape((1, -1) + (1,) * n), out.shape))
    return out


def max_pool_grad_nd(x, gout, ksize, stride=None, pad=0, cover_all=False):
    """NativeMaxPoolGradKernel over n spatial axes (pool.cc:97-143): ArgMax of the windows (padding holds the lowest value; native tie
    rule), gout placed at that kernel offset of a zero col, Col2Im."""
    x, gout = np.asarray(x), np.asarray(gout)
    n = x.ndim - 2
    ksize = _tuple_n(ksize, n)
    stride = ksize if stride is None else _tuple_n(stride, n)
    pad = _tuple_n(pad, n)
    col = _windows_nd(x, ksize, stride, pad, cover_all, _lowest(x.dtype))
    idx = argmax(col, tuple(range(2, 2 + n)))
    taps = np.arange(int(np.prod(ksize))).reshape((1, 1) + ksize + (1,) * n)
    lift = (slice(None), slice(None)) + (None,) * n
    gcol = np.where(idx[lift] == taps, gout[lift], np.zeros((), x.dtype)).astype(x.dtype)
    return np.ascontiguousarray(_col2im_nd(gcol, stride, pad, x.shape[2:]))


def max_pool_grad_grad_nd(x, ggx, ksize, stride=None, pad=0, cover_all=False):
    """NativeMaxPoolGradGradKernel over n spatial axes (pool.cc:147-177): the element of every window of ggx at the ArgMax position
    of x's window (a position in the padding reads the lowest value)."""
    x, ggx = np.asarray(x), np.asarray(ggx)
    n = x.ndim - 2
    ksize = _tuple_n(ksize, n)
    stride = ksize if stride is None else _tuple_n(stride, n)
    pad = _tuple_n(pad, n)
    idx = argmax(_windows_nd(x, ksize, stride, pad, cover_all, _lowest(x.dtype)), tuple(range(2, 2 + n)))
    col = _windows_nd(ggx, ksize, stride, pad, cover_all, _lowest(x.dtype))
    col = np.moveaxis(col, tuple(range(2, 2 + n)), tuple(range(2 + n, 2 + 2 * n)))  # kernel axes last
    flat = col.reshape(col.shape[:2 + n] + (-1,))
    return np.take_along_axis(flat, idx[..., None], axis=-1)[..., 0]


def average_pool_grad_nd(x, gout, ksize, stride=None, pad=0, pad_mode='ignore'):
    """NativeAveragePoolGradKernel over n spatial axes (pool.cc:304-346): gout (divided by the windows' widths first in 'ignore'
    mode) broadcast over the kernel axes, Col2Im, divided by the window size afterwards in 'zero' mode."""
    x, gout = np.asarray(x), np.asarray(gout)
    n = x.ndim - 2
    ksize = _tuple_n(ksize, n)
    stride = ksize if stride is None else _tuple_n(stride, n)
    pad = _tuple_n(pad, n)
    g = gout
    if pad_mode == 'ignore':
        widths = None
        for i in range(n):
            d, k, st, p = x.shape[2 + i], ksize[i], stride[i], pad[i]
            start = np.arange(gout.shape[2 + i]).astype(x.dtype) * _scalar_as(st, x.dtype) - _scalar_as(p, x.dtype)
            end = start + _scalar_as(k, x.dtype)
            w = (np.minimum(end, _scalar_as(d, x.dtype)) - np.maximum(start, _scalar_as(0, x.dtype))).astype(x.dtype)
            widths = w if widths is None else (widths[..., None] * w).astype(x.dtype)
        g = divide(gout, np.broadcast_to(widths, gout.shape))
    lift = (slice(None), slice(None)) + (None,) * n
    gcol = np.broadcast_to(g[lift], gout.shape[:2] + ksize + gout.shape[2:])
    gx = np.ascontiguousarray(_col2im_nd(gcol, stride, pad, x.shape[2:]))
    if pad_mode == 'zero':
        gx = divide(gx, _scalar_as(int(np.prod(ksize)), x.dtype))
    return gx


def take(a, indices, axis, mode=None):
    """NativeTakeKernel (indexing.cc:31-103): mode None/'raise' raise IndexError when out of range."""
    a = np.asarray(a)
    idx = np.asarray(indices).astype(np.int64)
    dim = a.shape[axis]
    if mode in (None, 'raise'):
        if ((idx < -dim) | (idx >= dim)).any():
            raise IndexError('Index is out of bounds for axis %d with size %d' % (axis, dim))
        idx = np.where(idx < 0, idx + dim, idx)
    elif mode == 'wrap':
        idx = np.where(idx < 0, dim - ((-idx + dim - 1) % dim + 1), idx % dim)
    elif mode == 'clip':
        idx = np.clip(idx, 0, dim - 1)
    else:
        raise ValueError(mode)
    return np.take(a, idx, axis=axis)


def lstm(c, x):
    """Lstm (CX/routines/connection.cc:396-446): gate k of unit j sits at column 4j+k."""
    c, x = np.asarray(c), np.asarray(x)
    g = x.reshape(x.shape[0], x.shape[1] // 4, 4)
    a = tanh(g[:, :, 0])
    i = sigmoid(g[:, :, 1])
    f = sigmoid(g[:, :, 2])
    o = sigmoid(g[:, :, 3])
    new_c = add(multiply(a, i), multiply(f, c))
    h = multiply(o, tanh(new_c))
    return h, new_c


def _math(x):
    """GetMathResultDtype: float dtypes stay, everything else computes in float32 (CX/routines/type_util.h)."""
    x = np.asarray(x)
    return x if x.dtype.kind == 'f' else x.astype(np.float32)


def clipped_relu(x, z):
    """Minimum(Maximum(0, x), z) = IfGreaterElse(max, z, z, max) (CX/routines/activation.cc:51-55, misc.cc)."""
    m = relu(_math(x))
    zz = _scalar_as(z, m.dtype)
    return np.where(m > zz, zz, m).astype(m.dtype)


def crelu(x, axis=1):
    """Relu(Concatenate({x, -x}, axis)) (CX/routines/activation.cc:57-64)."""
    x = _math(x)
    return relu(np.concatenate([x, multiply(x, _scalar_as(-1, x.dtype))], axis))


def elu(x, alpha=1.0):
    """Where(x > 0, x, alpha * Expm1(x)) (CX/routines/activation.cc:66-72)."""
    x = _math(x)
    return where(x > 0, x, multiply(expm1(x), _scalar_as(alpha, x.dtype)), x.dtype)


def leaky_relu(x, slope=0.2):
    """Where(x >= 0, x, slope * x) (CX/routines/activation.cc:86-92)."""
    x = _math(x)
    return where(x >= 0, x, multiply(x, _scalar_as(slope, x.dtype)), x.dtype)


def softplus(x, beta=1.0):
    """(Maximum(beta*x, 0) + Log1p(Exp(-Fabs(beta*x)))) * (1/beta) (CX/routines/activation.cc:151-158)."""
    x = _math(x)
    bx = multiply(x, _scalar_as(beta, x.dtype))
    neg_abs = multiply(absolute(bx), _scalar_as(-1, x.dtype))
    return multiply(add(relu(bx), log1p(exp(neg_abs))), _scalar_as(1.0 / beta, x.dtype))


def tree_lstm(*arrays):
    """TreeLstm(c_1..c_n, x) -> (c, h), gate-major gates a, i, o, f_1..f_n (CX/routines/activation.cc:94-121)."""
    cs, x = [np.asarray(a) for a in arrays[:-1]], np.asarray(arrays[-1])
    n = 3 + len(cs)
    g = x.reshape((x.shape[0], n, x.shape[1] // n) + x.shape[2:])
    a, i, o = tanh(g[:, 0]), sigmoid(g[:, 1]), sigmoid(g[:, 2])
    fs = [sigmoid(g[:, 3 + k]) for k in range(len(cs))]
    acc = multiply(cs[0], fs[0])
    for k in range(1, len(cs)):
        acc = add(acc, multiply(cs[k], fs[k]))
    c = add(multiply(a, i), acc)
    return c, multiply(o, tanh(c))


def slstm(c_prev1, c_prev2, x1, x2):
    """SLstm -> (c, h), unit-major gates a, i, f, o (CX/routines/activation.cc:123-149)."""
    def gates(x):
        x = np.asarray(x)
        g = x.reshape((x.shape[0], x.shape[1] // 4, 4) + x.shape[2:])
        return g[:, :, 0], g[:, :, 1], g[:, :, 2], g[:, :, 3]
    a1, i1, f1, o1 = gates(x1)
    a2, i2, f2, o2 = gates(x2)
    a1, i1, f1 = tanh(a1), sigmoid(i1), sigmoid(f1)
    a2, i2, f2 = tanh(a2), sigmoid(i2), sigmoid(f2)
    o = sigmoid(add(o1, o2))
    c = add(add(add(multiply(a1, i1), multiply(a2, i2)), multiply(f1, c_prev1)), multiply(f2, c_prev2))
    return c, multiply(o, tanh(c))


def _stack_weight(ws):
    """StackWeight (CX/routines/n_step_rnn.cc:41-54)."""
    w = np.stack([np.asarray(a) for a in ws], 1)
    return w.reshape((w.shape[0] * w.shape[1],) + w.shape[2:])


def _gru_step(x, h, c, ws, bs, activation):
    """GruImpl (CX/routines/n_step_rnn.cc:56-86)."""
    gx = linear(x, np.concatenate(ws[0:3], 0), np.concatenate(bs[0:3], 0))
    gh = linear(h, np.concatenate(ws[3:6], 0), np.concatenate(bs[3:6], 0))
    u = gx.shape[1] // 3
    r = sigmoid(add(gx[:, :u], gh[:, :u]))
    z = sigmoid(add(gx[:, u:2 * u], gh[:, u:2 * u]))
    h_bar = tanh(add(gx[:, 2 * u:], multiply(r, gh[:, 2 * u:])))
    one_minus_z = add(multiply(z, _scalar_as(-1, z.dtype)), _scalar_as(1, z.dtype))  # Subtract(Scalar, Array) = Add(-Array, Scalar)
    return [add(multiply(one_minus_z, h_bar), multiply(z, h))]


def _lstm_step(x, h, c, ws, bs, activation):
    """LstmImpl (CX/routines/n_step_rnn.cc:88-110): cuDNN order i, f, c, o becomes the Lstm routine's a, i, f, o."""
    xw = _stack_weight([ws[2], ws[0], ws[1], ws[3]])
    hw = _stack_weight([ws[6], ws[4], ws[5], ws[7]])
    xb = _stack_weight([bs[2], bs[0], bs[1], bs[3]])
    hb = _stack_weight([bs[6], bs[4], bs[5], bs[7]])
    return list(lstm(c, add(linear(x, xw, xb), linear(h, hw, hb))))


def _rnn_step(x, h, c, ws, bs, activation):
    """RnnImpl (CX/routines/n_step_rnn.cc:112-139)."""
    s = add(linear(x, ws[0], bs[0]), linear(h, ws[1], bs[1]))
    return [tanh(s) if activation == 'tanh' else relu(s)]


def _one_direction(step, xs, h, c, ws, bs, activation):
    """OneDirectionalLoop (CX/routines/n_step_rnn.cc:141-194): only the first len(x) rows of the state advance."""
    h = np.array(h)
    c = None if c is None else np.array(c)
    hs = []
    for x in xs:
        n = x.shape[0]
        if n > h.shape[0]:
            raise ValueError('The batch size of x must be equal to or less than the size of state')
        out = step(x, h[:n], None if c is None else c[:n], ws, bs, activation)
        hs.append(out[0])
        h = np.concatenate([out[0], h[n:]], 0)
        if c is not None:
            c = np.concatenate([out[1], c[n:]], 0)
    return h, c, hs


def _n_step(step, n_layers, hx, cx, ws, bs, xs, bidirectional, activation=None):
    """NStepRnnImpl, the non-cuDNN branch (CX/routines/n_step_rnn.cc:360-429)."""
    d = 2 if bidirectional else 1
    hx = np.asarray(hx)
    cx = None if cx is None else np.asarray(cx)
    xs = [np.asarray(x) for x in xs]
    hy, cy = [], []
    for layer in range(n_layers):
        i = d * layer
        h, c, fw = _one_direction(step, xs, hx[i], None if cx is None else cx[i], ws[i], bs[i], activation)
        hy.append(h)
        cy.append(c)
        if bidirectional:
            i += 1
            h, c, bw = _one_direction(step, xs[::-1], hx[i], None if cx is None else cx[i], ws[i], bs[i], activation)
            bw = bw[::-1]
            hy.append(h)
            cy.append(c)
            xs = [np.concatenate([f, b], 1) for f, b in zip(fw, bw)]
        else:
            xs = fw
    if cx is not None:
        return np.stack(hy, 0), np.stack(cy, 0), xs
    return np.stack(hy, 0), xs


def n_step_lstm(n_layers, hx, cx, ws, bs, xs):
    return _n_step(_lstm_step, n_layers, hx, cx, ws, bs, xs, False)


def n_step_bilstm(n_layers, hx, cx, ws, bs, xs):
    return _n_step(_lstm_step, n_layers, hx, cx, ws, bs, xs, True)


def n_step_gru(n_layers, hx, ws, bs, xs):
    return _n_step(_gru_step, n_layers, hx, None, ws, bs, xs, False)


def n_step_bigru(n_layers, hx, ws, bs, xs):
    return _n_step(_gru_step, n_layers, hx, None, ws, bs, xs, True)


def n_step_rnn(n_layers, hx, ws, bs, xs, activation='tanh'):
    return _n_step(_rnn_step, n_layers, hx, None, ws, bs, xs, False, activation)


def n_step_birnn(n_layers, hx, ws, bs, xs, activation='tanh'):
    return _n_step(_rnn_step, n_layers, hx, None, ws, bs, xs, True, activation)


def _linalg_dtype(*arrays):
    dt = np.result_type(*[np.asarray(a).dtype for a in arrays])
    if dt == np.float16:
        raise TypeError('Half-precision (float16) is not supported')
    return dt if dt.kind == 'f' else (np.dtype(np.float32) if dt.itemsize < 8 else np.dtype(np.float64))


def solve(a, b):
    """SolveKernel: LAPACK gesv in the result dtype (CX/native/native_device/linalg.cc:280-311) -- numpy.linalg.solve is the same
    routine.  Raises numpy.linalg.LinAlgError where the native backend throws ChainerxError (info != 0)."""
    dt = _linalg_dtype(a, b)
    return np.linalg.solve(np.asarray(a).astype(dt), np.asarray(b).astype(dt)).astype(dt)


def inv(a):
    """InverseKernel: getrf + getri (CX/native/native_device/linalg.cc:313-347)."""
    dt = _linalg_dtype(a)
    a = np.asarray(a).astype(dt)
    return np.linalg.inv(a).astype(dt) if a.size else a.copy()


def cholesky(a):
    """CholeskyKernel: potrf on the lower triangle, strict upper triangle zero (CX/native/native_device/linalg.cc:560-600)."""
    dt = _linalg_dtype(a)
    a = np.asarray(a).astype(dt)
    return np.linalg.cholesky(np.tril(a) + np.tril(a, -1).T).astype(dt) if a.size else a.copy()


def eigh(a, uplo='L'):
    """SyevdKernel with compute_v: LAPACK syevd on the `uplo` triangle of the row-major matrix, eigenvalues ascending, eigenvectors
    as columns (CX/native/native_device/linalg.cc:602-660; routine CX/routines/linalg.cc:452-495) -- numpy.linalg.eigh calls the same
    driver.  Only floating-point input (VisitFloatingPointDtype)."""
    a = np.asarray(a)
    if a.dtype.kind != 'f' or a.dtype == np.float16:
        raise TypeError('eigh needs float32 / float64')
    if a.size == 0:
        return np.empty((0,), a.dtype), a.copy()
    w, v = np.linalg.eigh(a, UPLO=uplo.upper())
    return w.astype(a.dtype), v.astype(a.dtype)


def eigvalsh(a, uplo='L'):
    """SyevdKernel without compute_v (CX/routines/linalg.cc:497-511)."""
    return eigh(a, uplo)[0]


def qr(a, mode='reduced'):
    """QrKernel: LAPACK geqrf, then orgqr for 'reduced' / 'complete' (CX/native/native_device/linalg.cc:349-430; shapes per mode
    CX/routines/linalg.cc:333-366) -- numpy.linalg.qr drives the same two routines.  Returns (q, r), r for 'r', (h, tau) for 'raw'."""
    a = np.asarray(a)
    if a.dtype.kind != 'f' or a.dtype == np.float16:
        raise TypeError('qr needs float32 / float64')
    return np.linalg.qr(a, mode=mode)


def svd(a, full_matrices=True, compute_uv=True):
    """SvdKernel: LAPACK gesdd, job 'A' / 'S' / 'N' (CX/native/native_device/linalg.cc:432-503; shapes CX/routines/linalg.cc:194-228)
    -- numpy.linalg.svd calls the same driver.  Full u / vt of an empty matrix are identities (:445-452)."""
    a = np.asarray(a)
    if a.dtype.kind != 'f' or a.dtype == np.float16:
        raise TypeError('svd needs float32 / float64')
    return np.linalg.svd(a, full_matrices=full_matrices, compute_uv=compute_uv)


def pinv(a, rcond=1e-15):
    """PseudoInverse (CX/routines/linalg.cc:303-331): from the reduced SVD, singular values <= rcond * max(s) dropped; rcond is a
    C float in the binding (CX/python/routines.cc:444-448)."""
    a = np.asarray(a)
    u, s, vt = svd(a, full_matrices=False)
    if a.size == 0:
        return a.T.copy()
    cutoff = (np.float32(rcond) * s.max()).astype(a.dtype)
    sinv = np.where(s <= cutoff, 0, 1 / s).astype(a.dtype)
    return ((vt.T * sinv) @ u.T).astype(a.dtype)


def softmax_cross_entropy(x, t):
    """chainer/functions/loss/softmax_cross_entropy.py:123-130 (reduce='mean', normalize=True)."""
    x, t = np.asarray(x), np.asarray(t)
    score = log_softmax(x, 1)
    mask = (t[:, None] == np.arange(score.shape[1], dtype=t.dtype)).astype(score.dtype)
    num = sum(multiply(score, mask))
    den = sum(mask)
    return multiply(num, divide(_scalar_as(-1, score.dtype), den))

"""Pins of the CPU oracle (oracle/native.py + oracle/native_oracle.c).

The oracle is only trusted as far as it is pinned here.  Kinds of pin used, per function:

  R  literal input/expected vectors held by the reference's own tests (tests/golden/reference_vectors.json and
     the literals of tests/chainerx_tests/unit_tests/routines_tests/test_sorting.py:11-29, expected = numpy.argmax)
  X  the reference's own float16.cc compiled from the reference tree into oracle/_ref (when present)
  C  closed form / invariant in float64 or exact integer arithmetic
  L  an independent library routine (numpy, scipy)
  B  brute-force loops on small inputs, written from the definition of the operation (not from the oracle's code)

What stays "parity unpinned" at bit level (tolerance level is pinned): the float summation order of Sum, the float
bit patterns of the naive Dot, and ArgMax's tie rule between different 32-element blocks -- all three are derived from
the reference's source (CX/native/reduce.h:46-83, CX/native/native_device/dot.cc:181-227) and no vector held by the
reference distinguishes them from other orders.
"""
import ctypes
import itertools
import json
import math
import os

import numpy as np
import pytest
import scipy.special

from oracle import native as O
from helpers import padded, assert_close, assert_exact

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = json.load(open(os.path.join(HERE, 'golden', 'reference_vectors.json')))['cases']
REF_F16 = os.path.join(os.path.dirname(HERE), 'oracle', '_ref', 'libcxfloat16.so')


def build_input(spec, dtype):
    shape = spec['shape']
    pad = spec.get('padding', 0)
    if 'linear' in spec:
        start, step = spec['linear']
        return padded(shape, None, pad, dtype, start, step)
    return padded(shape, spec['data'], pad, dtype)


def norm_axis(axis):
    return None if axis is None else tuple(axis)


def run_golden(F, case, to_dev=lambda a: a, to_host=np.asarray):
    """Evaluates one golden case with routine namespace F; shared by the CPU (oracle) and GPU (hip) golden tests."""
    dt = np.dtype(case['dtype'])
    op = case['op']
    if op in ('sum', 'amax', 'amin'):
        x = build_input(case['input'], dt)
        axis = norm_axis(case['axis'])
        axis = None if axis is None else tuple(a % x.ndim for a in axis)
        out = getattr(F, op)(to_dev(x), axis, case['keepdims'])
    elif op in ('argmax', 'argmin'):
        x = build_input(case['input'], dt)
        axis = norm_axis(case['axis'])
        out = getattr(F, op)(to_dev(x), None if axis is None else axis[0])
    elif op == 'dot':
        out = F.dot(to_dev(build_input(case['a'], dt)), to_dev(build_input(case['b'], dt)))
    elif op == 'take':
        a = build_input(case['input'], dt)
        idx = np.asarray(case['indices']['data'], np.int64).reshape(case['indices']['shape'])
        out = F.take(to_dev(a), to_dev(idx), case['axis'], case['mode'])
    elif op in ('add', 'subtract', 'multiply', 'divide'):
        out = getattr(F, op)(to_dev(build_input(case['a'], dt)), to_dev(build_input(case['b'], dt)))
    elif op.endswith('_scalar'):
        a = to_dev(build_input(case['a'], dt))
        s = case['scalar']
        name = op[:-len('_scalar')]
        if F is O:
            out = getattr(F, name)(a, np.asarray(s, dt))
        else:
            out = getattr(F, name)(a, s)
    else:
        raise AssertionError('unknown golden op %s' % op)
    return to_host(out)


@pytest.mark.parametrize('case', GOLDEN, ids=[c['name'] for c in GOLDEN])
def test_oracle_matches_reference_vectors(case):
    """R: every literal vector the reference's C++ tests hold for these kernels (cite in the JSON)."""
    got = run_golden(O, case)
    exp = np.asarray(case['expected'])
    shape = tuple(case.get('expected_shape', got.shape))
    assert got.shape == shape
    assert np.array_equal(got.reshape(-1).astype(np.float64), exp.reshape(-1).astype(np.float64))


# ---------------------------------------------------------------------------------------------
# float16
# ---------------------------------------------------------------------------------------------
def _f32_samples():
    rng = np.random.default_rng(16)
    bits = rng.integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32)
    rand = bits.view(np.float32)
    near_half = np.arange(0, 1 << 16, dtype=np.uint16).view(np.float16).astype(np.float32)
    # neighbours of every representable half and of every rounding midpoint
    mids = (near_half[:-1].astype(np.float64) + near_half[1:].astype(np.float64)) / 2
    with np.errstate(all='ignore'):
        mids = mids[np.isfinite(mids)].astype(np.float32)
    edge = np.concatenate([near_half, np.nextafter(near_half, np.float32(np.inf)), np.nextafter(near_half, np.float32(-np.inf)),
                           mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                           np.array([65504, 65519.99, 65520, 65536, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 2.9802326e-8, 6.1e-5], np.float32)])
    return np.concatenate([rand, edge, -edge])


def test_float16_conversions_match_numpy():
    """L: numpy's float16 uses the same npy_floatbits_to_halfbits algorithm the reference says it borrowed
    (CX/float16.cc:24-26).  Exhaustive half->float, 1.5M sampled/edge float->half."""
    allh = np.arange(1 << 16, dtype=np.uint16)
    assert_exact(O.half_bits_to_float(allh), allh.view(np.float16).astype(np.float32))
    x = _f32_samples()
    got = O.float_to_half_bits(x)
    with np.errstate(all='ignore'):
        ref = x.astype(np.float16).view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], ref[~nan])
    assert (((got[nan] & 0x7c00) == 0x7c00) & ((got[nan] & 0x3ff) != 0)).all()  # NaN stays NaN
    assert np.array_equal(got[nan] & 0x8000, ref[nan] & 0x8000)


def test_float16_literals_of_reference_test():
    """R: CX/float16_test.cc:60-73 (zeros), :102-110 (infinities), :132-157 (round-to-nearest-even of 1 + 3*2^-11)."""
    f = np.array([0.0, -0.0, np.inf, -np.inf], np.float32)
    assert O.float_to_half_bits(f).tolist() == [0x0000, 0x8000, 0x7c00, 0xfc00]
    back = O.half_bits_to_float(np.array([0x0000, 0x8000, 0x7c00, 0xfc00], np.uint16))
    assert back[0] == 0 and not np.signbit(back[0]) and back[1] == 0 and np.signbit(back[1])
    assert back[2] == np.inf and back[3] == -np.inf
    # a value exactly between mantissas 1 and 2 rounds to the even one (2)
    tie = np.array([1.0 + 1.5 * 2.0 ** -10], np.float32)
    assert int(O.float_to_half_bits(tie)[0]) & 0x3ff == 0x2
    for bit in range(0x7c01, 0x8000, 37):  # NaN payloads stay NaN (:113-121)
        assert np.isnan(O.half_bits_to_float(np.array([bit, bit | 0x8000], np.uint16))).all()


@pytest.mark.skipif(not os.path.exists(REF_F16), reason='oracle/_ref/libcxfloat16.so not built (needs the reference tree)')
def test_float16_matches_compiled_reference():
    """X: chainerx::Float16 itself, compiled from the reference's float16.cc by oracle/Makefile."""
    ref = ctypes.CDLL(REF_F16)
    i64 = ctypes.c_int64
    u16p, f32p = ctypes.POINTER(ctypes.c_uint16), ctypes.POINTER(ctypes.c_float)
    allh = np.arange(1 << 16, dtype=np.uint16)
    out = np.empty(allh.size, np.float32)
    ref.ref_half_to_float(allh.ctypes.data_as(u16p), out.ctypes.data_as(f32p), i64(allh.size))
    assert_exact(O.half_bits_to_float(allh), out)
    x = np.ascontiguousarray(_f32_samples())
    hb = np.empty(x.size, np.uint16)
    ref.ref_float_to_half(x.ctypes.data_as(f32p), hb.ctypes.data_as(u16p), i64(x.size))
    assert np.array_equal(O.float_to_half_bits(x), hb)
    # Float16 arithmetic (operator+ and operator* via float) against the oracle's elementwise add / multiply
    rng = np.random.default_rng(7)
    a = rng.integers(0, 1 << 16, 1 << 18).astype(np.uint16)
    b = rng.integers(0, 1 << 16, 1 << 18).astype(np.uint16)
    for name, fn in (('ref_half_add', O.add), ('ref_half_mul', O.multiply)):
        r = np.empty(a.size, np.uint16)
        getattr(ref, name)(a.ctypes.data_as(u16p), b.ctypes.data_as(u16p), r.ctypes.data_as(u16p), i64(a.size))
        got = fn(a.view(np.float16), b.view(np.float16))
        both_nan = np.isnan(got) & np.isnan(r.view(np.float16))
        assert (both_nan | (got.view(np.uint16) == r)).all(), name


# ---------------------------------------------------------------------------------------------
# elementwise
# ---------------------------------------------------------------------------------------------
def test_elementwise_single_rounding():
    """C: each op is one IEEE operation in the array dtype; for float32 the float64 result rounded once is the same
    thing (a double holds the exact sum/product of two floats)."""
    rng = np.random.default_rng(1)
    a = rng.standard_normal(4096).astype(np.float32) * 100
    b = rng.standard_normal(4096).astype(np.float32)
    assert_exact(O.add(a, b), (a.astype(np.float64) + b.astype(np.float64)).astype(np.float32))
    assert_exact(O.subtract(a, b), (a.astype(np.float64) - b.astype(np.float64)).astype(np.float32))
    assert_exact(O.multiply(a, b), (a.astype(np.float64) * b.astype(np.float64)).astype(np.float32))
    # float16: Float16(float(a) op float(b))
    ah, bh = a.astype(np.float16), b.astype(np.float16)
    assert_exact(O.add(ah, bh), (ah.astype(np.float32) + bh.astype(np.float32)).astype(np.float16))
    assert_exact(O.multiply(ah, bh), (ah.astype(np.float32) * bh.astype(np.float32)).astype(np.float16))
    # bool: Add is OR, Multiply is AND (CX/arithmetic_ops.h:18-24)
    p, q = rng.random(64) > 0.5, rng.random(64) > 0.5
    assert np.array_equal(O.add(p, q), p | q) and np.array_equal(O.multiply(p, q), p & q)


def test_relu_select_and_nan():
    """C: IfLessElse(x, 0, 0, x): negative -> 0, NaN < 0 is false so NaN passes through (misc.cc:39-61)."""
    x = np.array([-1.5, -0.0, 0.0, 2.0, np.nan, -np.inf, np.inf], np.float32)
    got = O.relu(x)
    assert np.array_equal(got[[0, 2, 3, 5, 6]], np.array([0, 0, 2, 0, np.inf], np.float32))
    assert np.isnan(got[4]) and got[1] == 0
    xi = np.array([-3, 0, 7], np.int8)
    assert_exact(O.relu(xi), np.array([0, 0, 7], np.int8))


def test_math_functions_within_ulps():
    """L: exp/log/tanh/sqrt are libm calls in the reference (CX/numeric.h:55-87); compare with float64 libm."""
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(20000) * 3).astype(np.float32)
    for name in ('exp', 'tanh'):
        ref = getattr(np, name)(x.astype(np.float64))
        got = getattr(O, name)(x).astype(np.float64)
        assert np.abs(got - ref).max() <= 2 * np.spacing(np.abs(ref).astype(np.float32)).max()
    xp = np.abs(x) + np.float32(1e-3)
    assert_close(O.log(xp), np.log(xp.astype(np.float64)).astype(np.float32), 1e-6)
    assert_exact(O.sqrt(xp), np.sqrt(xp.astype(np.float64)).astype(np.float32))  # sqrt is correctly rounded
    assert_close(O.sigmoid(x), scipy.special.expit(x.astype(np.float64)).astype(np.float32), 1e-6)


# ---------------------------------------------------------------------------------------------
# reductions
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize('dtype', ['float32', 'float64', 'float16', 'int32', 'int8', 'uint8', 'bool'])
@pytest.mark.parametrize('shape,axis', [((5, 70), 1), ((5, 70), 0), ((3, 4, 5), (0, 2)), ((2, 1031), None), ((2, 3, 150), (1, 2))])
def test_sum_integer_valued_is_exact(dtype, shape, axis):
    """C: with small integer values every partial sum is exact, whatever the order; int/bool inputs sum to int64
    (CX/routines/reduction.cc:34-49)."""
    rng = np.random.default_rng(3)
    x = rng.integers(0, 2, shape).astype(dtype) if dtype == 'bool' else rng.integers(0 if dtype == 'uint8' else -4, 5, shape).astype(dtype)
    got = O.sum(x, axis)
    ref = x.astype(np.int64).sum(axis)
    assert got.dtype == (np.int64 if np.dtype(dtype).kind in 'biu' else np.dtype(dtype))
    assert np.array_equal(got.astype(np.int64), ref)
    assert O.sum(x, axis, True).shape == x.astype(np.int64).sum(axis, keepdims=True).shape


def test_sum_float_within_pairwise_bound():
    """C: |pairwise sum - exact| <= eps * (log2(n)+8) * sum|x| (any 4x8xtree order obeys it; a serial sum of 1M terms
    would not, in general).  fp16 accumulates in float32 and rounds once (reduction.cc:105)."""
    rng = np.random.default_rng(4)
    for n in (7, 32, 33, 1000, 65536, 1 << 20):
        x = rng.standard_normal((3, n)).astype(np.float32)
        got = O.sum(x, 1).astype(np.float64)
        exact = np.array([math.fsum(r) for r in x.astype(np.float64)])
        bound = np.finfo(np.float32).eps * (math.log2(n) + 8) * np.abs(x).astype(np.float64).sum(1)
        assert (np.abs(got - exact) <= bound).all(), n
    xh = rng.standard_normal((4, 5000)).astype(np.float16)
    exact = np.array([math.fsum(r) for r in xh.astype(np.float64)])
    got = O.sum(xh, 1)
    assert got.dtype == np.float16
    assert np.abs(got.astype(np.float64) - exact).max() <= np.abs(exact).max() * 2.0 ** -10 + 0.05


def test_amax_matches_numpy_and_propagates_nan():
    """L + C: order independent; NaN propagates (statistics.cc:38-42) like numpy.max."""
    rng = np.random.default_rng(5)
    for dt in ('float32', 'float64', 'float16', 'int16', 'uint8', 'int64'):
        x = (rng.standard_normal((6, 7, 40)) * 50).astype(dt)
        for axis in (0, 2, (0, 2), None):
            assert_exact(O.amax(x, axis), np.asarray(x.max(axis)))
    x = rng.standard_normal((5, 100)).astype(np.float32)
    x[1, 3] = np.nan
    x[4, 99] = np.nan
    with np.errstate(all='ignore'):
        assert_exact(O.amax(x, 1), x.max(1))


SORTING_LITERALS = [  # tests/chainerx_tests/unit_tests/routines_tests/test_sorting.py:11-29, valid params
    (np.asarray(0), None), (np.asarray(-1), None), (np.asarray(float('inf')), None), (np.asarray(float('nan')), None),
    (np.asarray(-float('inf')), None), (np.asarray([4, 1, 4, 1]), None), (np.asarray([4, 1, 4, 1]), 0),
    (np.asarray([[4, 4, 1, 1], [4, 1, 4, 1]]), 0), (np.asarray([[4, 4, 1, 1], [4, 1, 4, 1]]).T, 1), (np.asarray([-2, -3, -1]), 0),
    (np.asarray([-0.0, +0.0, +0.0, -0.0]), None), (np.asarray([[True, True, False, False], [True, False, True, False]]), 0),
    (np.ones((2, 3)), 1), (np.ones((2, 3)), -2),
]


@pytest.mark.parametrize('x,axis', SORTING_LITERALS, ids=[str(i) for i in range(len(SORTING_LITERALS))])
def test_argmax_reference_literals(x, axis):
    """R: the reference's argmax test takes numpy.argmax as the expected value on these inputs."""
    for dt in ([x.dtype] if x.dtype == np.bool_ else [np.float32, np.float64, np.float16, np.int32]):
        if np.dtype(dt).kind != 'f' and not np.isfinite(np.asarray(x, np.float64)).all():
            continue
        xa = x.astype(dt)
        got = O.argmax(xa, axis)
        assert got.dtype == np.int64
        assert np.array_equal(got, np.argmax(xa, axis))


def test_argmax_tie_free_and_in_block_ties():
    """C: without ties the answer is unique (= numpy.argmax); ties inside one 32-element block and in the <=3-element
    tail resolve to the first index like numpy (reduce.h:28-31,65,69-72).  The rule between blocks: test_argmax_block_tie_literals."""
    rng = np.random.default_rng(6)
    for n in (1, 5, 31, 32, 33, 100, 4096, 70001):
        x = rng.permutation(n * 3).reshape(3, n).astype(np.float32)
        assert np.array_equal(O.argmax(x, 1), x.argmax(1))
        assert np.array_equal(O.argmax(x.T.copy(), 0), x.argmax(1))
    x = rng.integers(0, 3, (200, 32)).astype(np.float32)  # many ties, single block
    assert np.array_equal(O.argmax(x, 1), x.argmax(1))
    x = rng.integers(0, 3, (200, 35)).astype(np.float32)
    x[:, :32] -= 10  # maximum lives in the 3-element tail
    assert np.array_equal(O.argmax(x, 1), x.argmax(1))


def block_tie_rows(dtype, lo=-50, hi=40):
    """(name, row, expected argmax, mirrored row whose argmin is the same index) for every hand-traced case of
    tests/golden/argmax_block_ties.json: the maximum at the listed positions, distinct smaller values elsewhere."""
    cases = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'argmax_block_ties.json')))['cases']
    rows = []
    for c in cases:
        n = c['length']
        rng = np.random.default_rng(n * 7 + len(c['max_at']))
        row = rng.integers(lo, hi, n).astype(np.float64)
        row[c['max_at']] = hi + 3
        rows.append((c['name'], row.astype(dtype), c['expected'], (-row).astype(dtype)))
    return rows


def test_argmax_block_tie_literals():
    """R-by-hand: the tie rule between 32-element blocks (the later block wins), traced through the reference's
    PairwiseReduction in tests/golden/README.md; a first-index-wins (numpy) or last-index-wins rule fails several cases."""
    numpy_rule = last_rule = 0
    for dt in (np.float32, np.float16, np.float64, np.int32, np.int8):
        for name, row, expected, mirrored in block_tie_rows(dt):
            assert int(O.argmax(row, 0)) == expected, (name, dt)
            assert int(O.argmin(mirrored, 0)) == expected, (name, dt)
            m = np.stack([row, row[::-1].copy(), row])  # as rows of a matrix, and as a column of its transpose
            assert int(O.argmax(m, 1)[0]) == expected and int(O.argmax(m, 1)[2]) == expected, (name, dt)
            assert int(O.argmax(np.ascontiguousarray(m.T), 0)[0]) == expected, (name, dt)
            numpy_rule += int(np.argmax(row)) != expected
            last_rule += (len(row) - 1 - int(np.argmax(row[::-1]))) != expected
    assert numpy_rule > 0 and last_rule > 0  # the fixture tells the rule apart from both simple ones


def test_argmax_nan_rule():
    """C from the functor (reduction.cc:44-52): replace iff accum.argmax < 0 or accum.max < next.max, so a NaN never
    replaces a number, and a leading NaN is never replaced (inside one block, where visiting order is index order)."""
    x = np.array([[1, np.nan, 3, 2], [np.nan, 5, 6, 7], [np.nan, np.nan, np.nan, np.nan]], np.float32)
    assert O.argmax(x, 1).tolist() == [2, 0, 0]


def test_log_softmax_matches_scipy():
    rng = np.random.default_rng(8)
    for dt, tol in (('float32', 2e-6), ('float64', 1e-14)):
        x = (rng.standard_normal((37, 1000)) * 4).astype(dt)
        ref = scipy.special.log_softmax(x.astype(np.float64), axis=1)
        got = O.log_softmax(x, 1)
        assert got.dtype == np.dtype(dt)
        assert np.abs(got - ref).max() / np.abs(ref).max() <= tol
        assert np.allclose(np.exp(got.astype(np.float64)).sum(1), 1, atol=1e-5)  # rows are distributions
        assert_close(O.log_softmax(x + np.asarray(3, dt), 1), got, 1e-5 if dt == 'float32' else 1e-12)  # shift invariance


def test_softmax_cross_entropy_closed_form():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((100, 10)).astype(np.float32)
    t = rng.integers(0, 10, 100).astype(np.int32)
    ref = -scipy.special.log_softmax(x.astype(np.float64), axis=1)[np.arange(100), t].mean()
    assert abs(float(O.softmax_cross_entropy(x, t)) - ref) <= 1e-6 * abs(ref)


# ---------------------------------------------------------------------------------------------
# dot / conv
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize('dtype,tol', [('float32', 2e-6), ('float64', 1e-14), ('float16', 2e-3)])
def test_dot_matches_float64_matmul(dtype, tol):
    """L: numpy float64 matmul; integer-valued operands give the exact result."""
    rng = np.random.default_rng(10)
    for m, k, n in ((7, 33, 5), (64, 64, 64), (100, 784, 50), (1, 1, 1)):
        a = rng.standard_normal((m, k)).astype(dtype)
        b = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(dtype)
        ref = a.astype(np.float64) @ b.astype(np.float64)
        got = O.dot(a, b)
        assert got.dtype == np.dtype(dtype)
        assert np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30) <= tol
        ai = rng.integers(-3, 4, (m, k)).astype(dtype)
        bi = rng.integers(-3, 4, (k, n)).astype(dtype)
        assert np.array_equal(O.dot(ai, bi).astype(np.int64), ai.astype(np.int64) @ bi.astype(np.int64))


INT_DTYPES = ('int8', 'uint8', 'int16', 'int32', 'int64')


def wrap_to(value, dtype):
    """A Python integer reduced to the two's-complement range of `dtype`."""
    info = np.iinfo(dtype)
    value &= (1 << info.bits) - 1
    return value - (1 << info.bits) if info.min < 0 and value >= 1 << (info.bits - 1) else value


def test_dot_of_integers_and_bool_wraps_like_one_accumulator():
    """L: the native loop acc = a*b + acc with an accumulator of the array dtype (dot.cc:130-134, 200-214), evaluated with Python's
    unbounded integers and reduced modulo 2^bits, over the full value range of every integer dtype (a sum kept in a wider type
    or saturated fails); bool is "any of the conjunctions"."""
    rng = np.random.default_rng(12)
    for dtype in INT_DTYPES:
        info = np.iinfo(dtype)
        a = rng.integers(info.min, info.max, (5, 9), dtype=dtype, endpoint=True)
        b = rng.integers(info.min, info.max, (9, 4), dtype=dtype, endpoint=True)
        got = O.dot(a, b)
        assert got.dtype == np.dtype(dtype)
        for i in range(5):
            for j in range(4):
                acc = sum(int(a[i, l]) * int(b[l, j]) for l in range(9))
                assert int(got[i, j]) == wrap_to(acc, dtype), (dtype, i, j)
    a = rng.integers(0, 2, (6, 7)).astype(bool)
    b = rng.integers(0, 4, (7, 5)) == 0
    got = O.dot(a, b)
    assert got.dtype == np.bool_
    want = [[any(a[i, l] and b[l, j] for l in range(7)) for j in range(5)] for i in range(6)]
    assert np.array_equal(got, np.array(want))


def brute_conv(x, w, b, stride, pad, cover_all):
    """Definition of the cross-correlation (float64), out extent from the definition of cover_all: the last window must
    cover the last padded input element (chainer.utils.conv.get_conv_outsize)."""
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    sh, sw = stride
    ph, pw = pad

    def out_dim(d, k, s, p):
        if cover_all:
            return (d + 2 * p - k + s - 1) // s + 1
        return (d + 2 * p - k) // s + 1
    OH, OW = out_dim(H, R, sh, ph), out_dim(W, S, sw, pw)
    out = np.zeros((N, K, OH, OW))
    x = x.astype(np.float64)
    w = w.astype(np.float64)
    for n, k, oh, ow in itertools.product(range(N), range(K), range(OH), range(OW)):
        acc = 0.0
        for c, r, s in itertools.product(range(C), range(R), range(S)):
            ih, iw = oh * sh - ph + r, ow * sw - pw + s
            if 0 <= ih < H and 0 <= iw < W:
                acc += x[n, c, ih, iw] * w[k, c, r, s]
        out[n, k, oh, ow] = acc + (float(b[k]) if b is not None else 0.0)
    return out


CONV_GRID = [  # the 2-D rows of the reference's grid, tests/.../routines_tests/test_connection.py:183-203
    ((2, 3, 4, 4), (2, 3, 3, 3), False, (2, 2), (2, 0)),
    ((2, 3, 4, 4), (2, 3, 3, 3), True, (1, 1), (0, 0)),
    ((1, 3, 4, 4), (2, 3, 3, 3), True, (1, 2), (1, 1)),
    ((1, 3, 4, 4), (2, 3, 3, 3), True, (2, 2), (2, 0)),
    ((2, 5, 7, 6), (4, 5, 1, 1), True, (2, 2), (0, 0)),
    ((1, 2, 9, 9), (3, 2, 7, 7), False, (2, 2), (3, 3)),
]


@pytest.mark.parametrize('xs,ws,bias,stride,pad', CONV_GRID)
@pytest.mark.parametrize('cover_all', [False, True])
@pytest.mark.parametrize('dtype,tol', [('float32', 2e-6), ('float64', 1e-14), ('float16', 2e-3)])
def test_conv_matches_brute_force(xs, ws, bias, stride, pad, cover_all, dtype, tol):
    rng = np.random.default_rng(11)
    x = rng.standard_normal(xs).astype(dtype)
    w = (rng.standard_normal(ws) / np.sqrt(np.prod(ws[1:]))).astype(dtype)
    b = rng.standard_normal(ws[0]).astype(dtype) if bias else None
    ref = brute_conv(x, w, b, stride, pad, cover_all)
    got = O.conv(x, w, b, stride, pad, cover_all)
    assert got.shape == ref.shape and got.dtype == np.dtype(dtype)
    assert np.abs(got - ref).max() / np.abs(ref).max() <= tol


def test_conv_out_dim_formula():
    """C: CX/routines/connection.cc:37-49."""
    assert O.conv_out_dim(224, 7, 2, 3, False) == 112
    assert O.conv_out_dim(112, 3, 2, 1, False) == 56
    assert O.conv_out_dim(112, 3, 2, 0, False) == 55
    assert O.conv_out_dim(112, 3, 2, 0, True) == 56
    assert O.conv_out_dim(4, 3, 2, 2, False) == 3
    with pytest.raises(ValueError):
        O.conv_out_dim(2, 5, 1, 0, False)


def test_linear_is_dot_with_transposed_weight_plus_bias():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((9, 4, 5)).astype(np.float32)
    w = rng.standard_normal((7, 20)).astype(np.float32)
    b = rng.standard_normal(7).astype(np.float32)
    ref = x.reshape(9, 20).astype(np.float64) @ w.T.astype(np.float64) + b
    assert_close(O.linear(x, w, b), ref.astype(np.float32), 2e-6)


# ---------------------------------------------------------------------------------------------
# normalization / pooling / indexing / lstm
# ---------------------------------------------------------------------------------------------
BN_GRID = [  # tests/.../routines_tests/test_normalization.py:50-58 (<= 4-D rows)
    ((3, 2), (2,), None), ((5, 4, 3, 2), (4, 3, 2), None), ((5, 4, 3, 2), (4, 3, 2), (0,)), ((5, 4, 3, 2), (4,), (0, 2, 3)),
]


@pytest.mark.parametrize('xs,rs,axis', BN_GRID)
@pytest.mark.parametrize('dtype,tol', [('float32', 2e-6), ('float64', 1e-14), ('float16', 4e-3)])
def test_fixed_batch_norm_closed_form(xs, rs, axis, dtype, tol):
    rng = np.random.default_rng(13)
    x = rng.standard_normal(xs).astype(dtype)
    g, b, m = [rng.standard_normal(rs).astype(dtype) for _ in range(3)]
    v = rng.uniform(0.5, 1.5, rs).astype(dtype)
    axes = (0,) if axis is None else axis
    red = tuple(1 if i in axes else d for i, d in enumerate(xs))
    g64, b64, m64, v64 = [p.astype(np.float64).reshape(red) for p in (g, b, m, v)]
    ref = (x.astype(np.float64) - m64) / np.sqrt(v64 + 2e-5) * g64 + b64
    got = O.fixed_batch_norm(x, g, b, m, v, 2e-5, axis)
    assert got.dtype == np.dtype(dtype) and got.shape == x.shape
    assert np.abs(got - ref).max() / np.abs(ref).max() <= tol


POOL_GRID = [  # 2-D rows of tests/.../routines_tests/test_pooling.py:15-27,121-133
    ((2, 3, 4, 4), (3, 3), (1, 1), (0, 0)), ((2, 3, 4, 4), (3, 3), None, (0, 0)), ((1, 3, 4, 4), (3, 3), (1, 2), (1, 1)),
    ((1, 3, 4, 4), (3, 3), (2, 2), (2, 0)), ((2, 4, 9, 8), (3, 2), (2, 1), (1, 0)),
]


def brute_pool(x, ksize, stride, pad, cover_all, mode):
    N, C, H, W = x.shape
    kh, kw = ksize
    sh, sw = stride if stride is not None else ksize
    ph, pw = pad
    ex_h = sh - 1 if cover_all else 0
    ex_w = sw - 1 if cover_all else 0
    OH = (H + 2 * ph - kh + ex_h) // sh + 1
    OW = (W + 2 * pw - kw + ex_w) // sw + 1
    out = np.zeros((N, C, OH, OW))
    for n, c, oh, ow in itertools.product(range(N), range(C), range(OH), range(OW)):
        vals = []
        for r, s in itertools.product(range(kh), range(kw)):
            ih, iw = oh * sh - ph + r, ow * sw - pw + s
            if 0 <= ih < H and 0 <= iw < W:
                vals.append(float(x[n, c, ih, iw]))
        if mode == 'max':
            out[n, c, oh, ow] = max(vals) if vals else -np.inf
        elif mode == 'zero':
            out[n, c, oh, ow] = sum(vals) / (kh * kw)
        else:
            out[n, c, oh, ow] = sum(vals) / len(vals) if vals else np.nan
    return out


@pytest.mark.parametrize('xs,ksize,stride,pad', POOL_GRID)
@pytest.mark.parametrize('dtype', ['float32', 'float64', 'float16'])
def test_pooling_matches_brute_force(xs, ksize, stride, pad, dtype):
    rng = np.random.default_rng(14)
    x = rng.standard_normal(xs).astype(dtype)
    for cover_all in (False, True):
        ref = brute_pool(x, ksize, stride, pad, cover_all, 'max')
        got = O.max_pool(x, ksize, stride, pad, cover_all)
        assert got.dtype == x.dtype and np.array_equal(got.astype(np.float64), ref)  # max is exact
    tol = {'float32': 2e-6, 'float64': 1e-14, 'float16': 3e-3}[dtype]
    for mode in ('zero', 'ignore'):
        ref = brute_pool(x, ksize, stride, pad, False, mode)
        got = O.average_pool(x, ksize, stride, pad, mode).astype(np.float64)
        fin = np.isfinite(ref)
        assert np.abs(got[fin] - ref[fin]).max() <= tol * max(1.0, np.abs(ref[fin]).max())


def test_take_modes():
    """L + B: numpy.take for in-range / wrap / clip; out-of-range raises in the default mode (indexing.cc:68-74)."""
    rng = np.random.default_rng(15)
    a = rng.integers(-100, 100, (6, 5, 4)).astype(np.int16)
    idx = rng.integers(-5, 5, (3, 2))
    for axis in (0, 1, 2):
        dim = a.shape[axis]
        ii = np.clip(idx, -dim, dim - 1)
        assert_exact(O.take(a, ii, axis), np.take(a, ii, axis=axis))
        big = idx * 7
        assert_exact(O.take(a, big, axis, 'wrap'), np.take(a, big, axis=axis, mode='wrap'))
        assert_exact(O.take(a, big, axis, 'clip'), np.take(a, np.clip(big, 0, dim - 1), axis=axis))
    with pytest.raises(IndexError):
        O.take(a, np.array([6]), 0)
    with pytest.raises(IndexError):
        O.take(a, np.array([-7]), 0, 'raise')


def test_lstm_closed_form():
    """C: gate k of unit j at column 4j+k; a=tanh, i,f,o=sigmoid; c' = a*i + f*c; h = o*tanh(c') (connection.cc:396-446)."""
    rng = np.random.default_rng(17)
    c = rng.standard_normal((5, 6))
    x = rng.standard_normal((5, 24))
    a, i, f, o = [x[:, k::4] for k in range(4)]
    sig = scipy.special.expit
    c_ref = np.tanh(a) * sig(i) + sig(f) * c
    h_ref = sig(o) * np.tanh(c_ref)
    for dt, tol in (('float64', 1e-14), ('float32', 1e-6)):
        h, cn = O.lstm(c.astype(dt), x.astype(dt))
        assert np.abs(h - h_ref).max() <= tol and np.abs(cn - c_ref).max() <= tol


def test_power_integer_rule_brute_force():
    """B: chainerx::Power on integers (CX/numeric.h:85-125) equals exact integer exponentiation reduced modulo 2^bits for
    non-negative exponents, and the 1 / -1 / 0 rule for negative ones -- checked for every int8 base against Python's pow."""
    bases = np.arange(-128, 128, dtype=np.int8)
    for e in range(-4, 12):
        got = O.power(bases, np.full(bases.shape, e, np.int8))
        if e < 0:
            exp = np.array([1 if b == 1 else ((-1 if e % 2 else 1) if b == -1 else 0) for b in bases.tolist()], np.int8)
        else:
            exp = np.array([((pow(b, e) + 128) % 256) - 128 for b in bases.tolist()], np.int8)
        assert np.array_equal(got, exp), e
    ub = np.arange(0, 256, dtype=np.uint8)
    for e in range(0, 10):
        assert np.array_equal(O.power(ub, np.full(ub.shape, e, np.uint8)), np.array([pow(b, e) % 256 for b in ub.tolist()], np.uint8))


def test_amin_argmin_mirror_amax_argmax():
    """C: minimum = -maximum of the negated data with the same tree, so tie-free data must agree with numpy, a NaN
    propagates, and the ArgMin literals of the reference (array_test.cc:1436-1454, in the golden file) hold."""
    rng = np.random.default_rng(31)
    x = rng.standard_normal((9, 777)).astype(np.float32)
    assert np.array_equal(O.amin(x, 1), x.min(axis=1))
    assert np.array_equal(O.argmin(x, 1), x.argmin(axis=1))
    xi = rng.integers(-2 ** 62, 2 ** 62, (5, 99))
    assert np.array_equal(O.amin(xi, 1), xi.min(axis=1))
    for dt in ('int8', 'uint8', 'bool'):
        xs = (rng.integers(0, 2, (4, 50)) if dt == 'bool' else rng.integers(0, 100, (4, 50))).astype(dt)
        assert np.array_equal(O.amin(xs, 1), xs.min(axis=1)) and O.amin(xs, 1).dtype == xs.dtype
    x[3, 5] = np.nan
    assert np.isnan(O.amin(x, 1)[3]) and not np.isnan(O.amin(x, 1)[2])
    # earlier index wins a tie inside a block, like argmax
    t = np.array([[3.0, 1.0, 1.0, 2.0]], np.float32)
    assert O.argmin(t, 1)[0] == 1


def test_sign_abs_where_literals():
    """C: closed forms.  Sign: NaN passes, zero of either sign gives zero; Abs wraps at the lowest integer; Where selects."""
    x = np.array([-2.5, -0.0, 0.0, 3.0, np.nan, -np.inf], np.float32)
    s = O.sign(x)
    assert np.array_equal(s[:4], [-1, 0, 0, 1]) and np.isnan(s[4]) and s[5] == -1
    assert np.array_equal(O.absolute(np.array([-128, -1, 127], np.int8)), np.array([-128, 1, 127], np.int8))
    assert np.array_equal(O.absolute(np.array([200, 3], np.uint8)), np.array([200, 3], np.uint8))
    assert np.array_equal(O.where(np.array([1, 0, 2]), np.array([1, 2, 3]), 9, 'int32'), np.array([1, 9, 3], np.int32))
    assert np.array_equal(O.logical_xor(np.array([0, 2, 0, 5]), np.array([0, 0, 3, 7])), [False, True, True, False])


def test_floor_divide_mod_brute_force():
    """B: for every pair of int8 values the oracle equals Python's // and % (floor semantics, sign of the divisor), with the
    reference's conventions for zero operands (native/native_device/arithmetic.cc:107-139, 260-295); floats against
    math.floor(x / y) and Python's % on exactly representable operands."""
    a = np.arange(-128, 128, dtype=np.int8)
    x, y = np.meshgrid(a, a, indexing='ij')
    keep = ~((x == -128) & (y == -1))  # lowest / -1 overflows in the reference as well
    xs, ys = x[keep], y[keep]
    fd = np.array([0 if q == 0 else p // q for p, q in zip(xs.tolist(), ys.tolist())], np.int8)
    md = np.array([0 if (p == 0 or q == 0) else p % q for p, q in zip(xs.tolist(), ys.tolist())], np.int8)
    assert np.array_equal(O.floor_divide(xs, ys), fd)
    assert np.array_equal(O.mod(xs, ys), md)
    u = np.arange(0, 256, dtype=np.uint8)
    ux, uy = [v.reshape(-1) for v in np.meshgrid(u, u, indexing='ij')]
    assert np.array_equal(O.floor_divide(ux, uy), np.array([0 if q == 0 else p // q for p, q in zip(ux.tolist(), uy.tolist())], np.uint8))
    f = np.array([-7.5, -3.0, -0.5, 0.0, 0.5, 2.25, 7.0, 10.75], np.float32)
    fx, fy = [v.reshape(-1) for v in np.meshgrid(f, f[f != 0], indexing='ij')]
    assert np.array_equal(O.floor_divide(fx, fy), np.array([np.floor(p / q) for p, q in zip(fx.tolist(), fy.tolist())], np.float32))
    assert np.array_equal(O.mod(fx, fy), np.array([p % q for p, q in zip(fx.tolist(), fy.tolist())], np.float32))
    assert np.isnan(O.mod(np.float32([1.0]), np.float32([0.0]))[0])


def test_cumsum_add_at_closed_forms():
    """C: on integer-valued data any order is exact, so Cumsum must equal numpy.cumsum and AddAt numpy.add.at; the last
    prefix of a float Cumsum is the strictly serial sum (CX/native/reduce.h:98-113), checked against a Python loop."""
    rng = np.random.default_rng(34)
    x = rng.integers(-50, 50, (6, 40)).astype(np.float32)
    assert np.array_equal(O.cumsum(x, 1), np.cumsum(x, axis=1))
    assert O.cumsum(np.array([True, True, False]), 0).dtype == np.int64
    y = rng.standard_normal(500).astype(np.float32)
    acc = np.float32(0)
    for v in y:
        acc = np.float32(acc + v)
    assert O.cumsum(y, 0)[-1] == acc
    a = rng.integers(-9, 9, (4, 5, 3)).astype(np.int32)
    idx = np.array([[0, 4], [4, -1]])
    b = rng.integers(-9, 9, (4, 2, 2, 3)).astype(np.int32)
    ref = a.copy()
    np.add.at(ref, (slice(None), idx % 5), b)
    assert np.array_equal(O.add_at(a, idx, 1, b), ref)
    with pytest.raises(IndexError):
        O.add_at(a, np.array([5]), 1, b[:, :1, 0])
    # Linspace closed form: endpoints exact, interior from the reference's expression
    assert np.array_equal(O.linspace(0, 10, 11, True, 'float32'), np.arange(11, dtype=np.float32))
    assert O.linspace(2, 3, 1, True, 'float64')[0] == 2.0


# ---------------------------------------------------------------------------------------------
# backward / training kernels
# ---------------------------------------------------------------------------------------------
BACKWARD_CONV_CASES = [  # N, C, H, W, K, kh, kw, stride, pad, cover_all
    (2, 3, 6, 5, 4, 3, 3, (1, 1), (1, 1), False), (1, 2, 7, 7, 3, 3, 2, (2, 1), (0, 1), False),
    (2, 4, 5, 6, 2, 1, 1, (2, 2), (0, 0), False), (1, 3, 6, 6, 2, 3, 3, (2, 2), (1, 1), True),
]


@pytest.mark.parametrize('case', BACKWARD_CONV_CASES)
def test_conv_backward_adjoint_identities(case):
    """C: convolution is bilinear, so <conv(x, w), gy> = <x, conv_transpose(gy, w)> = <w, conv_grad_weight(x, gy)> exactly (up to
    float64 rounding).  A transposed operand, a flipped kernel or a wrong stride / pad offset breaks the identity."""
    N, C, H, W, K, kh, kw, st, pd, cv = case
    rng = np.random.default_rng(41)
    x = rng.standard_normal((N, C, H, W))
    w = rng.standard_normal((K, C, kh, kw))
    y = O.conv(x, w, None, st, pd, cv)
    gy = rng.standard_normal(y.shape)
    lhs = float((y * gy).sum())
    gx = O.conv_transpose(gy, w, None, st, pd, (H, W))
    assert gx.shape == x.shape
    assert abs(float((x * gx).sum()) - lhs) <= 1e-10 * max(1.0, abs(lhs))
    gw = O.conv_grad_weight(w.shape, x, gy, st, pd, cv)
    assert gw.shape == w.shape
    assert abs(float((w * gw).sum()) - lhs) <= 1e-10 * max(1.0, abs(lhs))
    if not cv:  # default out_size is the inverse of GetConvOutDim (CX/routines/connection.cc:51-56)
        exp = tuple(s * (d - 1) + k - 2 * p for d, k, s, p in zip(y.shape[2:], (kh, kw), st, pd))
        assert O.conv_transpose(gy, w, None, st, pd).shape[2:] == exp
    b = rng.standard_normal(C)
    assert np.allclose(O.conv_transpose(gy, w, b, st, pd, (H, W)), gx + b.reshape(1, -1, 1, 1), rtol=0, atol=1e-12)


def test_pool_backward_brute_force_and_adjoint():
    """B + C: MaxPoolGrad against a loop that routes every gout element to the first maximum of its window (the native ArgMax
    tie rule inside one window); AveragePoolGrad through the adjoint identity <avg_pool(x), g> = <x, avg_pool_grad(g)>."""
    rng = np.random.default_rng(42)
    for (shape, k, s, p, cv) in [((2, 3, 7, 6), (3, 3), (2, 2), (1, 1), False), ((1, 2, 5, 5), (2, 3), (1, 2), (0, 1), True),
                                 ((2, 1, 6, 6), (3, 3), (3, 3), (0, 0), False)]:
        x = rng.integers(-3, 4, shape).astype(np.float64)  # ties on purpose
        y = O.max_pool(x, k, s, p, cv)
        g = rng.standard_normal(y.shape)
        ref = np.zeros_like(x)
        N, C, H, W = shape
        for n in range(N):
            for c in range(C):
                for oh in range(y.shape[2]):
                    for ow in range(y.shape[3]):
                        best, pos = -np.inf, None
                        for r in range(k[0]):
                            for q in range(k[1]):
                                ih, iw = oh * s[0] - p[0] + r, ow * s[1] - p[1] + q
                                v = x[n, c, ih, iw] if 0 <= ih < H and 0 <= iw < W else -np.inf
                                if pos is None or v > best:
                                    best, pos = v, (ih, iw)
                        if 0 <= pos[0] < H and 0 <= pos[1] < W:
                            ref[n, c, pos[0], pos[1]] += g[n, c, oh, ow]
        assert np.allclose(O.max_pool_grad(x, g, k, s, p, cv), ref, rtol=0, atol=1e-12)
    for mode in ('zero', 'ignore'):
        for (shape, k, s, p) in [((2, 3, 7, 6), (3, 3), (2, 2), (1, 1)), ((1, 2, 8, 8), (2, 2), (2, 2), (0, 0)), ((1, 1, 5, 7), (3, 2), (1, 2), (1, 0))]:
            x = rng.standard_normal(shape)
            y = O.average_pool(x, k, s, p, mode)
            g = rng.standard_normal(y.shape)
            gx = O.average_pool_grad(x, g, k, s, p, mode)
            assert abs(float((y * g).sum()) - float((x * gx).sum())) <= 1e-10


def test_batch_norm_training_closed_forms():
    """C: normalised output has per-channel mean beta and variance gamma^2 * var/(var+eps); running statistics follow
    decay * old + (1 - decay) * batch (variance with n/(n-1)); the gradients agree with central differences in float64."""
    rng = np.random.default_rng(43)
    x = rng.standard_normal((4, 3, 5, 2)) * 2 + 1
    gamma, beta = rng.uniform(0.5, 1.5, 3), rng.standard_normal(3)
    rm, rv = rng.standard_normal(3), rng.uniform(0.5, 1.5, 3)
    eps, decay = 2e-5, 0.9
    out, nrm, nrv, state = O.batch_norm(x, gamma, beta, rm, rv, eps, decay)
    m, v = x.mean(axis=(0, 2, 3)), x.var(axis=(0, 2, 3))
    assert np.allclose(out.mean(axis=(0, 2, 3)), beta, atol=1e-12)
    assert np.allclose(out.var(axis=(0, 2, 3)), gamma ** 2 * v / (v + eps), atol=1e-12)
    n = 4 * 5 * 2
    assert np.allclose(nrm, decay * rm + (1 - decay) * m, atol=1e-14)
    assert np.allclose(nrv, decay * rv + (1 - decay) * v * n / (n - 1), atol=1e-14)
    gout = rng.standard_normal(x.shape)
    gx, gg, gb = O.batch_norm_grad(x, gamma, gout, state)
    loss = lambda xx, g_, b_: float((O.batch_norm(xx, g_, b_, rm, rv, eps, decay)[0] * gout).sum())
    h = 1e-6
    for idx in [(0, 0, 0, 0), (3, 2, 4, 1), (1, 1, 2, 0)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        assert abs((loss(xp, gamma, beta) - loss(xm, gamma, beta)) / (2 * h) - gx[idx]) <= 1e-6
    for c in range(3):
        e = np.zeros(3)
        e[c] = h
        assert abs((loss(x, gamma + e, beta) - loss(x, gamma - e, beta)) / (2 * h) - gg[c]) <= 1e-6
        assert abs((loss(x, gamma, beta + e) - loss(x, gamma, beta - e)) / (2 * h) - gb[c]) <= 1e-6


def _brute_conv_nd(x, w, b, stride, pad, cover_all, number=float):
    """Definition of the cross-correlation, one output element at a time, in float64 (or, with number=int, in Python's
    unbounded integers)."""
    n = x.ndim - 2
    od = [O.conv_out_dim(x.shape[2 + d], w.shape[2 + d], stride[d], pad[d], cover_all) for d in range(n)]
    out = np.zeros((x.shape[0], w.shape[0]) + tuple(od), dtype=np.float64 if number is float else object)
    for idx in np.ndindex(*out.shape):
        nb, k, o = idx[0], idx[1], idx[2:]
        acc = number(0)
        for c in range(x.shape[1]):
            for kidx in np.ndindex(*w.shape[2:]):
                i = tuple(o[d] * stride[d] - pad[d] + kidx[d] for d in range(n))
                if all(0 <= i[d] < x.shape[2 + d] for d in range(n)):
                    acc += number(x[(nb, c) + i]) * number(w[(k, c) + kidx])
        out[idx] = acc + (number(b[k]) if b is not None else number(0))
    return out


def _brute_pool_nd(x, ksize, stride, pad, cover_all, kind):
    n = x.ndim - 2
    od = [O.conv_out_dim(x.shape[2 + d], ksize[d], stride[d], pad[d], cover_all) for d in range(n)]
    out = np.zeros(x.shape[:2] + tuple(od))
    for idx in np.ndindex(*out.shape):
        vals = []
        for kidx in np.ndindex(*ksize):
            i = tuple(idx[2 + d] * stride[d] - pad[d] + kidx[d] for d in range(n))
            if all(0 <= i[d] < x.shape[2 + d] for d in range(n)):
                vals.append(float(x[idx[:2] + i]))
        if kind == 'max':
            out[idx] = max(vals) if vals else -np.inf
        elif kind == 'zero':
            out[idx] = np.sum(vals) / np.prod(ksize)
        else:
            # the divisor is the product of the per-axis overlaps min(start + k, extent) - max(start, 0), which the reference does not
            # clamp at zero (CX/native/native_device/pool.cc:197-225): a window wholly outside an axis gives a negative factor
            div = 1.0
            for d in range(n):
                start = idx[2 + d] * stride[d] - pad[d]
                div *= min(start + ksize[d], x.shape[2 + d]) - max(start, 0)
            with np.errstate(all='ignore'):
                out[idx] = np.float64(np.sum(vals)) / div
    return out


# the reference's own grids: tests/chainerx_tests/unit_tests/routines_tests/test_connection.py:178-203, test_pooling.py:15-27
CONV_ND_GRID = [((1, 3), (5, 3), 1, 0), ((1, 3, 4), (5, 3, 2), 3, 2), ((2, 3, 4), (5, 3, 1), 1, 0), ((2, 3, 4, 4), (2, 3, 3, 3), 2, (2, 0)),
                ((1, 3, 4, 4), (2, 3, 3, 3), (1, 2), 1), ((2, 3, 2, 6, 3), (2, 3, 1, 3, 2), (1, 2, 3), (2, 0, 1)),
                ((1, 3, 2, 6, 3), (2, 3, 1, 3, 2), 2, (2, 0, 1))]
POOL_ND_GRID = [((2, 3, 4), (1,), 1, 0), ((1, 3, 4), (2,), 3, 2), ((2, 3, 4, 4), (3, 3), 1, 0), ((1, 3, 4, 4), (3, 3), (1, 2), 1),
                ((1, 3, 4, 4), (3, 3), 2, (2, 0)), ((1, 3, 2, 6, 3), (1, 3, 2), 2, (2, 0, 1)), ((2, 3, 2, 6, 3), (1, 3, 2), (1, 2, 3), (2, 0, 1)),
                ((1, 3, 2, 6, 3, 2), (1, 3, 2, 2), 2, 2)]


def test_conv_and_pooling_over_n_axes():
    """The restatements for any number of spatial axes: equal to the 2-D ones (pinned above) bit for bit on 2-D input, and equal to
    the definition evaluated element by element on the reference's grids of 0-, 1-, 3- and 4-D cases (a wrong axis order in the
    window copy, a missing cover_all row or a divisor taken over the wrong axes fails)."""
    rng = np.random.default_rng(61)
    tup = lambda v, n: (v,) * n if isinstance(v, int) else tuple(v)
    for dt in ('float32', 'float16'):
        x = rng.standard_normal((2, 3, 7, 6)).astype(dt)
        w = rng.standard_normal((4, 3, 3, 2)).astype(dt)
        b = rng.standard_normal(4).astype(dt)
        for cv in (False, True):
            assert np.array_equal(O.conv_nd(x, w, b, (2, 1), (1, 0), cv), O.conv(x, w, b, (2, 1), (1, 0), cv))
            assert np.array_equal(O.max_pool_nd(x, (3, 2), (2, 1), (1, 0), cv), O.max_pool(x, (3, 2), (2, 1), (1, 0), cv))
        for mode in ('zero', 'ignore'):
            assert np.array_equal(O.average_pool_nd(x, (3, 2), (2, 1), (1, 0), mode), O.average_pool(x, (3, 2), (2, 1), (1, 0), mode), equal_nan=True)
    for xs, ws, stride, pad in CONV_ND_GRID:
        n = len(xs) - 2
        x, w, b = rng.standard_normal(xs), rng.standard_normal(ws), rng.standard_normal(ws[0])
        for cv in (False, True):
            for bias in (None, b):
                got = O.conv_nd(x, w, bias, stride, pad, cv)
                want = _brute_conv_nd(x, w, bias, tup(stride, n), tup(pad, n), cv)
                assert got.shape == want.shape and np.allclose(got, want, rtol=1e-12, atol=1e-12), (xs, ws, stride, pad, cv)
    # integer dtypes: the definition in exact integer arithmetic, reduced modulo 2^bits (values large enough to wrap)
    for dtype in INT_DTYPES:
        info = np.iinfo(dtype)
        lo, hi = max(info.min, -2 ** 20), min(info.max, 2 ** 20)
        for xs, ws, stride, pad in CONV_ND_GRID[::3]:
            n = len(xs) - 2
            x = rng.integers(lo, hi, xs).astype(dtype)
            w = rng.integers(lo, hi, ws).astype(dtype)
            b = rng.integers(lo, hi, ws[0]).astype(dtype)
            got = O.conv_nd(x, w, b, stride, pad, False)
            want = _brute_conv_nd(x, w, b, tup(stride, n), tup(pad, n), False, number=int)
            assert got.dtype == np.dtype(dtype) and got.shape == want.shape
            assert all(int(g) == wrap_to(int(v), dtype) for g, v in zip(got.ravel(), want.ravel())), (dtype, xs, ws)
    for xs, ks, stride, pad in POOL_ND_GRID:
        n = len(xs) - 2
        x = rng.standard_normal(xs)
        for cv in (False, True):
            got = O.max_pool_nd(x, ks, stride, pad, cv)
            assert np.array_equal(got, _brute_pool_nd(x, ks, tup(stride, n), tup(pad, n), cv, 'max')), (xs, ks, stride, pad, cv)
        for mode in ('zero', 'ignore'):
            got = O.average_pool_nd(x, ks, stride, pad, mode)
            want = _brute_pool_nd(x, ks, tup(stride, n), tup(pad, n), False, mode)
            assert got.shape == want.shape and np.allclose(got, want, rtol=1e-12, atol=1e-12, equal_nan=True), (xs, ks, stride, pad, mode)


def test_gradients_over_n_axes():
    """The backward restatements for any number of spatial axes: equal to the 2-D ones (pinned above) bit for bit on 2-D input; on
    the reference's 0-, 1-, 3- and 4-D grids the convolution gradients are the adjoints of the forward restatement in float64
    (<conv(x, w), gy> = <w, grad_weight> = <x, conv_transpose(gy, w)>: a transposed operand or a wrong stride / pad axis breaks the
    identity), average-pool gradients the adjoint of average pooling, and the max-pool gradients the definition on tie-free data
    (gx collects the gradient of every window whose largest element it is; the double backward reads ggx there)."""
    rng = np.random.default_rng(67)
    tup = lambda v, n: (v,) * n if isinstance(v, int) else tuple(v)
    for dt in ('float32', 'float16', 'float64'):
        x = rng.standard_normal((2, 3, 7, 6)).astype(dt)
        w = rng.standard_normal((4, 3, 3, 2)).astype(dt)
        wt = rng.standard_normal((3, 4, 3, 2)).astype(dt)
        b = rng.standard_normal(4).astype(dt)
        gy = rng.standard_normal(O.conv(x, w, None, (2, 1), (1, 0)).shape).astype(dt)
        assert np.array_equal(O.conv_grad_weight_nd(w.shape, x, gy, (2, 1), (1, 0)), O.conv_grad_weight(w.shape, x, gy, (2, 1), (1, 0)))
        assert np.array_equal(O.conv_transpose_nd(x, wt, b, (2, 1), (1, 0)), O.conv_transpose(x, wt, b, (2, 1), (1, 0)))
        for cv in (False, True):
            g = rng.standard_normal(O.max_pool(x, (3, 2), (2, 1), (1, 0), cv).shape).astype(dt)
            assert np.array_equal(O.max_pool_grad_nd(x, g, (3, 2), (2, 1), (1, 0), cv), O.max_pool_grad(x, g, (3, 2), (2, 1), (1, 0), cv))
            gg = rng.standard_normal(x.shape).astype(dt)
            assert np.array_equal(O.max_pool_grad_grad_nd(x, gg, (3, 2), (2, 1), (1, 0), cv), O.max_pool_grad_grad(x, gg, (3, 2), (2, 1), (1, 0), cv))
        for mode in ('zero', 'ignore'):
            g = rng.standard_normal(O.average_pool(x, (3, 2), (2, 1), (1, 0), mode).shape).astype(dt)
            assert np.array_equal(O.average_pool_grad_nd(x, g, (3, 2), (2, 1), (1, 0), mode), O.average_pool_grad(x, g, (3, 2), (2, 1), (1, 0), mode),
                                  equal_nan=True)
    for xs, ws, stride, pad in CONV_ND_GRID:
        n = len(xs) - 2
        x, w = rng.standard_normal(xs), rng.standard_normal(ws)
        for cv in (False, True):
            y = O.conv_nd(x, w, None, stride, pad, cv)
            gy = rng.standard_normal(y.shape)
            lhs = float((y * gy).sum())
            gw = O.conv_grad_weight_nd(ws, x, gy, stride, pad, cv)
            assert gw.shape == tuple(ws) and abs(float((gw * w).sum()) - lhs) <= 1e-10 * max(1.0, abs(lhs)), (xs, ws, stride, pad, cv)
            gx = O.conv_transpose_nd(gy, w, None, stride, pad, out_size=xs[2:])
            assert gx.shape == tuple(xs) and abs(float((gx * x).sum()) - lhs) <= 1e-10 * max(1.0, abs(lhs)), (xs, ws, stride, pad, cv)
        # the default output size and the bias of ConvTranspose: w read as [C_in, C_out, k...]
        wt = rng.standard_normal((xs[1], 4) + tuple(ws[2:]))
        st, pd = tup(stride, n), tup(pad, n)
        dims = tuple(s_ * (d - 1) + k - 2 * p_ for d, k, s_, p_ in zip(xs[2:], ws[2:], st, pd))
        if all(d > 0 for d in dims):
            bias = rng.standard_normal(4)
            out = O.conv_transpose_nd(x, wt, bias, stride, pad)
            assert out.shape == (xs[0], 4) + dims
            z = rng.standard_normal(out.shape)
            back = O.conv_nd(z, wt, None, stride, pad)  # the convolution whose adjoint this is
            lhs = float(((out - bias.reshape((1, 4) + (1,) * n)) * z).sum())
            assert back.shape == tuple(xs) and abs(float((back * x).sum()) - lhs) <= 1e-10 * max(1.0, abs(lhs)), (xs, ws, stride, pad)
    for xs, ks, stride, pad in POOL_ND_GRID:
        n = len(xs) - 2
        st, pd = tup(stride, n), tup(pad, n)
        x = rng.permutation(int(np.prod(xs))).reshape(xs).astype(np.float64)  # no ties
        for cv in (False, True):
            y = O.max_pool_nd(x, ks, stride, pad, cv)
            g = rng.standard_normal(y.shape)
            want = np.zeros(xs)
            ggx = rng.standard_normal(xs)
            want_gg = np.zeros(y.shape)
            for idx in np.ndindex(*y.shape):
                best = None
                for kidx in np.ndindex(*ks):
                    i = tuple(idx[2 + d] * st[d] - pd[d] + kidx[d] for d in range(n))
                    if all(0 <= i[d] < xs[2 + d] for d in range(n)):
                        pos = idx[:2] + i
                        if best is None or x[pos] > x[best]:
                            best = pos
                if best is None:  # a window entirely in the padding: its ArgMax is its first position, which lies outside x
                    want_gg[idx] = -np.inf
                    continue
                want[best] += g[idx]
                want_gg[idx] = ggx[best]
            got = O.max_pool_grad_nd(x, g, ks, stride, pad, cv)
            assert got.shape == tuple(xs) and np.allclose(got, want, rtol=1e-12, atol=1e-12), (xs, ks, stride, pad, cv)
            assert np.array_equal(O.max_pool_grad_grad_nd(x, ggx, ks, stride, pad, cv), want_gg), (xs, ks, stride, pad, cv)
        xr = rng.standard_normal(xs)
        for mode in ('zero', 'ignore'):
            y = O.average_pool_nd(xr, ks, stride, pad, mode)
            if not np.isfinite(y).all():
                continue  # windows that lie in the padding altogether divide by a width of zero
            g = rng.standard_normal(y.shape)
            gx = O.average_pool_grad_nd(xr, g, ks, stride, pad, mode)
            assert gx.shape == tuple(xs)
            lhs = float((y * g).sum())
            assert abs(float((gx * xr).sum()) - lhs) <= 1e-10 * max(1.0, abs(lhs)), (xs, ks, stride, pad, mode)


def test_batch_norm_dtypes():
    """The dtype rules of GenericBatchNormKernel (CX/routines/normalization.cc:176-193, 224-246).  float16 x with float32 parameters:
    computed in float32 -- statistics, state and running values are float32 and agree with the float64 closed form to float32
    accuracy, out / gx are float16 and within half a float16 ulp of it, and 50176 elements per channel are no problem.  All float16:
    the same size overflows the float16 Sum of (x - mean)^2 (native Sum hands out a float16, CX/native/native_device/reduction.cc:105-110):
    variance inf, inv_std 0, out == beta exactly."""
    rng = np.random.default_rng(44)
    shape = (64, 3, 28, 28)
    x = (rng.standard_normal(shape) * 2 + 0.5).astype(np.float16)
    gamma, beta = rng.uniform(0.5, 1.5, 3).astype(np.float32), rng.standard_normal(3).astype(np.float32)
    rm, rv = rng.standard_normal(3).astype(np.float32), rng.uniform(0.5, 1.5, 3).astype(np.float32)
    out, nrm, nrv, (mean, inv_std) = O.batch_norm(x, gamma, beta, rm, rv, 2e-5, 0.9)
    assert out.dtype == np.float16 and nrm.dtype == nrv.dtype == mean.dtype == inv_std.dtype == np.float32
    x64 = x.astype(np.float64)
    m, v = x64.mean(axis=(0, 2, 3)), x64.var(axis=(0, 2, 3))
    bc = lambda a: a.reshape(1, 3, 1, 1)
    assert np.allclose(mean.ravel(), m, rtol=1e-5, atol=1e-6) and np.allclose(inv_std.ravel(), 1 / np.sqrt(v + 2e-5), rtol=1e-5)
    want = (x64 - bc(m)) / np.sqrt(bc(v) + 2e-5) * bc(gamma.astype(np.float64)) + bc(beta.astype(np.float64))
    assert np.abs(out.astype(np.float64) - want).max() <= np.abs(want).max() * 2.0 ** -11 * 1.01  # one rounding to float16
    n = x.size // 3
    assert np.allclose(nrm, 0.9 * rm + 0.1 * m, rtol=1e-5, atol=1e-6) and np.allclose(nrv, 0.9 * rv + 0.1 * v * n / (n - 1), rtol=1e-5)
    gout = rng.standard_normal(shape).astype(np.float16)
    gx, gg, gb = O.batch_norm_grad(x, gamma, gout, (mean, inv_std))
    assert gx.dtype == np.float16 and gg.dtype == gb.dtype == np.float32
    g64 = gout.astype(np.float64)
    xh = (x64 - bc(m)) / np.sqrt(bc(v) + 2e-5)
    assert np.allclose(gb, g64.sum(axis=(0, 2, 3)), rtol=1e-4, atol=1e-3) and np.allclose(gg, (g64 * xh).sum(axis=(0, 2, 3)), rtol=1e-4, atol=1e-3)
    gx64 = bc(gamma.astype(np.float64)) / np.sqrt(bc(v) + 2e-5) * (g64 - (xh * bc((g64 * xh).sum(axis=(0, 2, 3))) + bc(g64.sum(axis=(0, 2, 3)))) / n)
    assert np.abs(gx.astype(np.float64) - gx64).max() <= np.abs(gx64).max() * 2.0 ** -10
    # all float16
    g16, b16 = gamma.astype(np.float16), beta.astype(np.float16)
    out, nrm, nrv, (mean, inv_std) = O.batch_norm(x, g16, b16, rm.astype(np.float16), rv.astype(np.float16), 2e-5, 0.9)
    assert out.dtype == nrm.dtype == mean.dtype == inv_std.dtype == np.float16
    assert np.all(inv_std == 0) and np.all(np.isinf(nrv)) and np.all(np.isfinite(mean))
    assert np.array_equal(out, np.broadcast_to(bc(b16), shape))


# ---------------------------------------------------------------------------------------------
# activations built from other routines, and the n-step recurrent family: textbook formulas in float64
# ---------------------------------------------------------------------------------------------
def _sig(v):
    return 1.0 / (1.0 + np.exp(-v))


def test_composed_activations_closed_forms():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((4, 6, 3)) * 3).astype(np.float32)
    x64 = x.astype(np.float64)
    assert np.allclose(O.clipped_relu(x, 2.5), np.clip(x64, 0, 2.5), rtol=1e-6)
    assert np.allclose(O.crelu(x, 1), np.concatenate([np.maximum(x64, 0), np.maximum(-x64, 0)], 1), rtol=1e-6)
    assert O.crelu(x, 2).shape == (4, 6, 6)
    assert np.allclose(O.elu(x, 0.7), np.where(x64 > 0, x64, 0.7 * (np.exp(x64) - 1)), rtol=1e-5, atol=1e-6)
    assert np.allclose(O.leaky_relu(x, 0.1), np.where(x64 >= 0, x64, 0.1 * x64), rtol=1e-6)
    assert np.allclose(O.softplus(x, 1.7), np.log1p(np.exp(1.7 * x64)) / 1.7, rtol=1e-5, atol=1e-6)
    assert O.elu(np.arange(-2, 3, dtype=np.int32)).dtype == np.float32  # integers compute in float32
    # TreeLstm with two children: gates are laid out gate-major (a | i | o | f1 | f2), unlike Lstm's unit-major layout
    c1, c2 = rng.standard_normal((2, 3, 5)).astype(np.float32)
    g = rng.standard_normal((3, 25)).astype(np.float32)
    a, i, o, f1, f2 = [g[:, k * 5:(k + 1) * 5].astype(np.float64) for k in range(5)]
    c_ref = np.tanh(a) * _sig(i) + c1 * _sig(f1) + c2 * _sig(f2)
    c, h = O.tree_lstm(c1, c2, g)
    assert np.allclose(c, c_ref, rtol=1e-5, atol=1e-6) and np.allclose(h, _sig(o) * np.tanh(c_ref), rtol=1e-5, atol=1e-6)
    # SLstm: unit-major gates (column 4*u + k), output gate from the sum of both inputs
    x1, x2 = rng.standard_normal((2, 3, 20)).astype(np.float32)
    ga = [x1[:, k::4].astype(np.float64) for k in range(4)]
    gb = [x2[:, k::4].astype(np.float64) for k in range(4)]
    c_ref = np.tanh(ga[0]) * _sig(ga[1]) + np.tanh(gb[0]) * _sig(gb[1]) + _sig(ga[2]) * c1 + _sig(gb[2]) * c2
    c, h = O.slstm(c1, c2, x1, x2)
    assert np.allclose(c, c_ref, rtol=1e-5, atol=1e-6)
    assert np.allclose(h, _sig(ga[3] + gb[3]) * np.tanh(c_ref), rtol=1e-5, atol=1e-6)


def _rnn_problem(rng, kind, n_layers, bidirectional, in_size=4, units=3, lengths=(5, 3, 3, 1)):
    """Random parameters and a batch of sequences sorted by decreasing length, time-major like the reference takes them."""
    nw = {'lstm': 8, 'gru': 6, 'rnn': 2}[kind]
    d = 2 if bidirectional else 1
    ws, bs = [], []
    for layer in range(n_layers):
        for _ in range(d):
            isz = in_size if layer == 0 else units * d
            ws.append([rng.uniform(-0.6, 0.6, (units, isz if j < nw // 2 else units)).astype(np.float32) for j in range(nw)])
            bs.append([rng.uniform(-0.3, 0.3, (units,)).astype(np.float32) for j in range(nw)])
    seqs = [rng.standard_normal((n, in_size)).astype(np.float32) for n in lengths]
    xs = [np.stack([s[t] for s in seqs if len(s) > t]) for t in range(max(lengths))]
    hx = rng.standard_normal((n_layers * d, len(lengths), units)).astype(np.float32)
    cx = rng.standard_normal((n_layers * d, len(lengths), units)).astype(np.float32)
    return ws, bs, seqs, xs, hx, cx


def _textbook_cell(kind, x, h, c, w, b, activation):
    """One step of one sequence, written from the gate equations (cuDNN / Chainer parameter order), float64."""
    w = [m.astype(np.float64) for m in w]
    b = [v.astype(np.float64) for v in b]
    if kind == 'lstm':
        i = _sig(w[0] @ x + b[0] + w[4] @ h + b[4])
        f = _sig(w[1] @ x + b[1] + w[5] @ h + b[5])
        g = np.tanh(w[2] @ x + b[2] + w[6] @ h + b[6])
        o = _sig(w[3] @ x + b[3] + w[7] @ h + b[7])
        c = f * c + i * g
        return o * np.tanh(c), c
    if kind == 'gru':
        r = _sig(w[0] @ x + b[0] + w[3] @ h + b[3])
        z = _sig(w[1] @ x + b[1] + w[4] @ h + b[4])
        n = np.tanh(w[2] @ x + b[2] + r * (w[5] @ h + b[5]))
        return (1 - z) * n + z * h, None
    s = w[0] @ x + b[0] + w[1] @ h + b[1]
    return (np.tanh(s) if activation == 'tanh' else np.maximum(s, 0)), None


def _textbook_n_step(kind, n_layers, bidirectional, ws, bs, seqs, hx, cx, activation='tanh'):
    """Every sequence on its own, in float64: layer by layer, forward in time and (bidirectional) backward from its own last step."""
    d = 2 if bidirectional else 1
    units = hx.shape[2]
    hy = np.zeros(hx.shape)
    cy = np.zeros(hx.shape)
    outs = []
    for bi, seq in enumerate(seqs):
        inp = seq.astype(np.float64)
        for layer in range(n_layers):
            per_dir = []
            for di in range(d):
                idx = layer * d + di
                h = hx[idx, bi].astype(np.float64)
                c = cx[idx, bi].astype(np.float64)
                hs = np.zeros((len(inp), units))
                order = range(len(inp)) if di == 0 else range(len(inp) - 1, -1, -1)
                for t in order:
                    h, c_new = _textbook_cell(kind, inp[t], h, c, ws[idx], bs[idx], activation)
                    c = c_new if c_new is not None else c
                    hs[t] = h
                hy[idx, bi] = h
                cy[idx, bi] = c
                per_dir.append(hs)
            inp = np.concatenate(per_dir, 1)
        outs.append(inp)
    T = max(len(s) for s in seqs)
    ys = [np.stack([o[t] for o in outs if len(o) > t]) for t in range(T)]
    return hy, cy, ys


@pytest.mark.parametrize('kind,n_layers,bidirectional,activation', [
    ('lstm', 1, False, None), ('lstm', 2, False, None), ('lstm', 2, True, None), ('gru', 1, False, None), ('gru', 2, True, None),
    ('rnn', 2, False, 'tanh'), ('rnn', 1, True, 'relu'), ('rnn', 2, True, 'tanh')])
def test_n_step_rnn_family_matches_textbook_recurrences(kind, n_layers, bidirectional, activation):
    """Pins the parameter order (which matrix feeds which gate), the stacking of gate rows, the handling of shrinking batches and
    the direction / layer wiring: a swapped gate, a transposed weight or a state row advanced past its sequence's end fails."""
    rng = np.random.default_rng(len(kind) * 100 + n_layers * 10 + int(bidirectional))
    ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, kind, n_layers, bidirectional)
    hy_ref, cy_ref, ys_ref = _textbook_n_step(kind, n_layers, bidirectional, ws, bs, seqs, hx, cx, activation or 'tanh')
    if kind == 'lstm':
        fn = O.n_step_bilstm if bidirectional else O.n_step_lstm
        hy, cy, ys = fn(n_layers, hx, cx, ws, bs, xs)
        assert np.allclose(cy, cy_ref, rtol=2e-5, atol=2e-6)
    elif kind == 'gru':
        fn = O.n_step_bigru if bidirectional else O.n_step_gru
        hy, ys = fn(n_layers, hx, ws, bs, xs)
    else:
        fn = O.n_step_birnn if bidirectional else O.n_step_rnn
        hy, ys = fn(n_layers, hx, ws, bs, xs, activation)
    assert hy.dtype == np.float32 and hy.shape == hx.shape
    assert np.allclose(hy, hy_ref, rtol=2e-5, atol=2e-6)
    assert len(ys) == len(ys_ref)
    for y, r in zip(ys, ys_ref):
        assert y.shape == r.shape and np.allclose(y, r, rtol=2e-5, atol=2e-6)


def test_n_step_rejects_a_growing_batch():
    rng = np.random.default_rng(0)
    ws, bs, seqs, xs, hx, cx = _rnn_problem(rng, 'rnn', 1, False)
    with pytest.raises(ValueError):
        O.n_step_rnn(1, hx[:, :2], ws, bs, xs)


def test_linalg_identities():
    """solve / inv / cholesky reduce to LAPACK routines through numpy; pinned by what defines them: a @ x = b, inv(a) @ a = I,
    L @ L.T = a with L lower triangular and only a's lower triangle read."""
    rng = np.random.default_rng(9)
    for n in (1, 2, 7, 40):
        a = rng.standard_normal((n, n)) + n * np.eye(n)
        b = rng.standard_normal((n, 3))
        for dt, tol in (('float64', 1e-11), ('float32', 2e-4)):
            x = O.solve(a.astype(dt), b.astype(dt))
            assert x.dtype == np.dtype(dt) and np.abs(a @ x - b).max() <= tol * n
            assert np.abs(O.solve(a.astype(dt), b[:, 0].astype(dt)) - x[:, 0]).max() <= tol
            assert np.abs(O.inv(a.astype(dt)) @ a - np.eye(n)).max() <= tol * n
            spd = (a @ a.T).astype(dt)
            lower = O.cholesky(spd)
            assert np.array_equal(lower, np.tril(lower)) and np.abs(lower @ lower.T - spd).max() <= tol * np.abs(spd).max() * n
            garbage_above = np.tril(spd) + np.triu(rng.standard_normal((n, n)).astype(dt), 1)
            assert np.array_equal(O.cholesky(garbage_above), lower)
    assert O.solve(np.eye(2, dtype=np.int32), np.ones(2, np.int32)).dtype == np.float32
    with pytest.raises(np.linalg.LinAlgError):
        O.solve(np.zeros((2, 2)), np.ones(2))
    with pytest.raises(np.linalg.LinAlgError):
        O.cholesky(-np.eye(2))


def test_eigh_identities():
    """eigh / eigvalsh reduce to LAPACK syevd through numpy; pinned by what defines them: a known spectrum (a = q diag(d) q.T) is
    recovered in ascending order, a @ v = v * w with orthonormal columns, and only the chosen triangle is read."""
    rng = np.random.default_rng(10)
    for n in (1, 2, 6, 30):
        q, _ = np.linalg.qr(rng.standard_normal((n, n)))
        d = np.sort(rng.standard_normal(n) * 3)
        a = (q * d) @ q.T
        a = (a + a.T) / 2
        for dt, tol in (('float64', 1e-12), ('float32', 1e-5)):
            ad = a.astype(dt)
            for uplo in ('U', 'l'):
                w, v = O.eigh(ad, uplo)
                assert w.dtype == np.dtype(dt) and v.dtype == np.dtype(dt)
                assert np.abs(w - d).max() <= tol * n * 10
                assert np.abs(ad.astype(np.float64) @ v - v * w).max() <= tol * n * 10
                assert np.abs(v.T.astype(np.float64) @ v - np.eye(n)).max() <= tol * n * 10
                noise = rng.standard_normal((n, n)).astype(dt)
                spoiled = np.triu(ad) + np.tril(noise, -1) if uplo.upper() == 'U' else np.tril(ad) + np.triu(noise, 1)
                assert np.array_equal(O.eigvalsh(spoiled, uplo), w)
    # a matrix whose two triangles differ: each triangle defines its own symmetric matrix
    m = np.array([[2., 1.], [0., 2.]])
    assert np.allclose(O.eigvalsh(m, 'U'), [1., 3.]) and np.allclose(O.eigvalsh(m, 'L'), [2., 2.])
    with pytest.raises(TypeError):
        O.eigh(np.eye(2, dtype=np.int32))


def test_qr_identities():
    """qr reduces to LAPACK geqrf / orgqr through numpy; pinned by what defines the factorisation: q @ r = a, orthonormal columns,
    r upper triangular with the shapes of each mode, and the raw form (reflector vectors + tau) rebuilding the same q by the
    Householder product H_0 H_1 ... with H_j = I - tau_j v_j v_j^T."""
    rng = np.random.default_rng(11)
    for m, n in ((1, 1), (4, 4), (7, 3), (3, 7), (20, 12)):
        a = rng.standard_normal((m, n))
        k = min(m, n)
        for dt, tol in (('float64', 1e-12), ('float32', 1e-5)):
            ad = a.astype(dt)
            q, r = O.qr(ad)
            assert q.shape == (m, k) and r.shape == (k, n) and q.dtype == np.dtype(dt)
            assert np.abs(q.astype(np.float64) @ r - ad).max() <= tol * 10 and np.array_equal(r, np.triu(r))
            assert np.abs(q.T.astype(np.float64) @ q - np.eye(k)).max() <= tol * 10
            qc, rc = O.qr(ad, 'complete')
            assert qc.shape == (m, m) and rc.shape == (m, n)
            assert np.abs(qc.astype(np.float64) @ rc - ad).max() <= tol * 10
            assert np.abs(qc.T.astype(np.float64) @ qc - np.eye(m)).max() <= tol * 10
            assert np.abs(qc[:, :k] - q).max() <= tol * 10 and np.abs(rc[:k] - r).max() <= tol * 10
            assert np.abs(O.qr(ad, 'r') - r).max() <= tol * 10
            h, tau = O.qr(ad, 'raw')
            assert h.shape == (n, m) and tau.shape == (k,)
            f = h.T.astype(np.float64)
            assert np.abs(np.triu(f)[:k] - r).max() <= tol * 10
            prod = np.eye(m)
            for j in range(k):
                v = np.zeros(m)
                v[j] = 1
                v[j + 1:] = f[j + 1:, j]
                prod = prod @ (np.eye(m) - tau[j] * np.outer(v, v))
            assert np.abs(prod[:, :k] - q).max() <= tol * 100
    with pytest.raises(TypeError):
        O.qr(np.eye(2, dtype=np.int64))


def test_svd_pinv_identities():
    """svd reduces to LAPACK gesdd through numpy; pinned by a prescribed decomposition (orthogonal factors and singular values
    chosen first, recovered afterwards), by u diag(s) vt = a with orthonormal factors in both shapes, and pinv by the four
    Moore-Penrose conditions and by the explicit inverse of a rank-deficient diagonal matrix."""
    rng = np.random.default_rng(12)
    for m, n in ((1, 1), (5, 5), (8, 3), (3, 8), (20, 13)):
        k = min(m, n)
        qu, _ = np.linalg.qr(rng.standard_normal((m, m)))
        qv, _ = np.linalg.qr(rng.standard_normal((n, n)))
        d = np.sort(rng.uniform(0.5, 4.0, k))[::-1]
        a = (qu[:, :k] * d) @ qv[:, :k].T
        for dt, tol in (('float64', 1e-12), ('float32', 1e-5)):
            ad = a.astype(dt)
            assert np.abs(O.svd(ad, compute_uv=False) - d).max() <= tol * 10
            for full in (True, False):
                u, s, vt = O.svd(ad, full_matrices=full)
                assert u.shape == (m, m if full else k) and s.shape == (k,) and vt.shape == (n if full else k, n)
                assert u.dtype == np.dtype(dt) and np.all(np.diff(s) <= 0) and np.abs(s - d).max() <= tol * 10
                assert np.abs((u[:, :k].astype(np.float64) * s) @ vt[:k] - ad).max() <= tol * 20
                assert np.abs(u.T.astype(np.float64) @ u - np.eye(u.shape[1])).max() <= tol * 20
                assert np.abs(vt.astype(np.float64) @ vt.T - np.eye(vt.shape[0])).max() <= tol * 20
            p = O.pinv(ad).astype(np.float64)
            assert p.shape == (n, m)
            for lhs, rhs in ((a @ p @ a, a), (p @ a @ p, p), ((a @ p).T, a @ p), ((p @ a).T, p @ a)):
                assert np.abs(lhs - rhs).max() <= tol * 200
    assert np.array_equal(O.pinv(np.diag([2., 0., 4.])), np.diag([0.5, 0., 0.25]))
    assert np.allclose(O.pinv(np.diag([2., 1e-3, 4.]), rcond=1e-2), np.diag([0.5, 0., 0.25]))
    u, s, vt = O.svd(np.zeros((0, 3), 'float32'))
    assert u.shape == (0, 0) and s.shape == (0,) and np.array_equal(vt, np.eye(3, dtype='float32'))
    assert O.pinv(np.zeros((0, 3))).shape == (3, 0)


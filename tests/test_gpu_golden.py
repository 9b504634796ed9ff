"""The reference's own literal vectors (tests/golden/reference_vectors.json) through the hip kernels."""
import numpy as np
import pytest

from test_oracle_pins import GOLDEN, run_golden, SORTING_LITERALS, block_tie_rows
from helpers import upload_view

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('case', GOLDEN, ids=[c['name'] for c in GOLDEN])
def test_hip_matches_reference_vectors(case):
    import chainer_amd as chx

    def to_dev(a):
        a = np.asarray(a)
        return upload_view(chx, a) if a.size else chx.array(a)

    got = run_golden(chx, case, to_dev, lambda o: o.get())
    exp = np.asarray(case['expected'])
    assert got.shape == tuple(case.get('expected_shape', got.shape))
    assert np.array_equal(got.reshape(-1).astype(np.float64), exp.reshape(-1).astype(np.float64))


@pytest.mark.parametrize('x,axis', SORTING_LITERALS, ids=[str(i) for i in range(len(SORTING_LITERALS))])
def test_argmax_reference_literals(x, axis):
    """tests/chainerx_tests/unit_tests/routines_tests/test_sorting.py:11-29: expected = numpy.argmax."""
    import chainer_amd as chx
    for dt in ([x.dtype] if x.dtype == np.bool_ else [np.float32, np.float64, np.float16, np.int32]):
        if np.dtype(dt).kind != 'f' and not np.isfinite(np.asarray(x, np.float64)).all():
            continue
        xa = np.ascontiguousarray(x.astype(dt))
        got = chx.argmax(upload_view(chx, x.astype(dt)) if x.ndim else chx.array(xa), axis).get()
        assert got.dtype == np.int64
        assert np.array_equal(got, np.argmax(xa, axis))


def test_argmax_block_tie_literals():
    """The hand-traced tie cases of tests/golden/argmax_block_ties.json (the later 32-element block wins; traces in
    tests/golden/README.md) through the hip ArgMax / ArgMin kernels: as a 1-D array (row kernel), as rows of a matrix, as a
    strided column (column kernels), and spread over a long row that is split across workgroups."""
    import chainer_amd as chx
    for dt in (np.float32, np.float16, np.float64, np.int32, np.int8):
        for name, row, expected, mirrored in block_tie_rows(dt):
            what = '%s %s' % (name, np.dtype(dt))
            assert int(chx.argmax(chx.array(row), 0).get()) == expected, what
            assert int(chx.argmin(chx.array(mirrored), 0).get()) == expected, what
            m = np.stack([row, row[::-1].copy(), row])
            got = chx.argmax(chx.array(m), 1).get()
            assert got[0] == expected and got[2] == expected, what
            assert int(chx.argmax(chx.array(np.ascontiguousarray(m.T)), 0).get()[0]) == expected, what
    # the same rule far out in a long row (blocks merged by the binary counter across workgroup boundaries): the oracle, itself
    # held to the literals above, is the reference here
    from oracle import native as O
    rng = np.random.default_rng(3)
    x = rng.integers(-100, 100, (3, 300000)).astype(np.float32)
    for r, positions in enumerate([(5, 40, 299999), (70000, 131072, 131073), (31, 32, 262144)]):
        x[r, list(positions)] = 1000
    assert np.array_equal(chx.argmax(chx.array(x), 1).get(), O.argmax(x, 1))
    assert np.array_equal(chx.argmin(chx.array(-x), 1).get(), O.argmin(-x, 1))

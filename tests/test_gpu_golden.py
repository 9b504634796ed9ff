"""The reference's own literal vectors (tests/golden/reference_vectors.json) through the hip kernels."""
import numpy as np
import pytest

from test_oracle_pins import GOLDEN, run_golden, SORTING_LITERALS
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

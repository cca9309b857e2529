"""The Reduce family through the C-ABI against the CPU restatement of the reference's loops.  Max and Min are bit-exact everywhere; sums
and products are bit-exact where the device runs the loop's order (one output per lane) and within 3e-5 of the sum of the magnitudes
where a wave reduces a long line as a tree (the loop's own rounding error is 7e-6 of that sum at 100000 elements)."""
import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import graph_runner as gr
from tests import util

pytestmark = pytest.mark.gpu

OPS = list(range(7))
CASES = [((1, 2, 3), [1]), ((3, 4), [0]), ((2, 3, 4), [1]), ((2, 3, 4), [-1]), ((2, 3, 4, 5), [1, 2]), ((4, 512), [1]), ((5, 7), None), ((6, 1, 5), [0, 2]),
         ((300, 70), [1]), ((64, 1000), [0]), ((3, 5000), [-1]), ((2, 17, 33), [1]), ((1, 100000), [1]), ((20000, 3), [1])]


@pytest.mark.parametrize("shape,axes", CASES)
def test_reduce_matches_the_reference_loops(rt, shape, axes):
    n = int(np.prod(shape))
    # magnitudes around 1 keep the products of up to 100000 factors inside the float range
    X = (np.float32(1) + np.float32(0.002) * util.normal(9801, n)).reshape(shape) * np.where(util.uniform01(9802, n) < 0.5, np.float32(-1), np.float32(1)).reshape(shape)
    be = gr.HipBackend(rt)
    outer, A, inner = ob.reduce_block(shape, axes)
    tree = inner == 1 and A >= 64 and outer < 16384
    for op in OPS:
        for keep in (1, 0):
            print("reduce", shape, axes, op, keep, flush=True)
            got, want = be.reduce(X, op, axes, keep), ob.reduce(X, op, axes, keep)
            assert got.shape == want.shape
            if op >= R.REDUCE_MAX or not tree:
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (op, np.abs(got - want).max())
            elif op == R.REDUCE_PROD:       # up to A roundings of 6e-8 each, in another order
                assert np.all(np.abs(got - want) <= (3e-7 * np.sqrt(A) + 1e-6) * np.abs(want))
            else:                           # the loop's own rounding grows with the line; the bound is relative to the sum of the magnitudes
                scale = {R.REDUCE_SUM: A, R.REDUCE_SUM_SQUARE: A, R.REDUCE_MEAN: 1.0, R.REDUCE_L2: np.sqrt(A)}[op]
                assert np.all(np.abs(got - want) <= 3e-5 * scale), (op, np.abs(got - want).max())
    assert np.abs(ob.reduce(X, R.REDUCE_MAX, axes, 0)).min() > 0.5


def test_reduce_literal_cases_of_the_reference_tests(rt):
    be = gr.HipBackend(rt)
    x = np.array([5, 2, 3, 5, 5, 4], np.float32).reshape(1, 2, 3)
    assert be.reduce(x, R.REDUCE_SUM, [0, 1, 2], 1).ravel().tolist() == [24.0]
    assert be.reduce(x, R.REDUCE_SUM_SQUARE, [2], 0).ravel().tolist() == [38.0, 66.0]
    assert be.reduce(x, R.REDUCE_MIN, [1], 0).ravel().tolist() == [5.0, 2.0, 3.0]
    assert be.reduce(x, R.REDUCE_MAX, [1], 0).ravel().tolist() == [5.0, 5.0, 4.0]
    assert be.reduce(np.arange(12, dtype=np.float32).reshape(3, 4), R.REDUCE_MEAN, [0], 0).tolist() == [4.0, 5.0, 6.0, 7.0]
    assert be.reduce(np.arange(24, dtype=np.float32).reshape(2, 3, 4), R.REDUCE_MEAN, [1], 0).ravel().tolist() == [4, 5, 6, 7, 16, 17, 18, 19]
    big = np.repeat(np.arange(1, 5, dtype=np.float32)[:, None], 512, axis=1)       # the reference's ReduceL2Large
    got = be.reduce(big, R.REDUCE_L2, [1], 0)
    assert np.all(np.abs(got - np.arange(1, 5) * np.sqrt(512.0)) <= 1e-5 * got)
    # NaN never wins `y < x`: Max and Min skip it as the reference's std::max / std::min do, a sum carries it
    nan = np.array([[1.0, np.nan, 3.0, -2.0]], np.float32)
    assert be.reduce(nan, R.REDUCE_MAX, [1], 0).tolist() == [3.0] and be.reduce(nan, R.REDUCE_MIN, [1], 0).tolist() == [-2.0]
    assert np.isnan(be.reduce(nan, R.REDUCE_SUM, [1], 0)[0])
    assert np.array_equal(be.reduce(nan, R.REDUCE_MAX, [1], 0), ob.reduce(nan, R.REDUCE_MAX, [1], 0))


def test_reduce_errors(rt):
    x = util.to_dev(np.zeros(8, np.float32))
    with pytest.raises(R.SofieHipError, match="unknown operator"):
        rt.call("sofie_hip_reduce_f32", util.ptr(x), util.ptr(x), 2, 4, 1, 7)
    with pytest.raises(R.SofieHipError, match="bad shape"):
        rt.call("sofie_hip_reduce_f32", util.ptr(x), util.ptr(x), 2, 0, 1, 0)
    with pytest.raises(R.SofieHipError, match="NULL"):
        rt.call("sofie_hip_reduce_f32", None, util.ptr(x), 2, 4, 1, 0)
    rt.call("sofie_hip_reduce_f32", None, None, 0, 4, 1, 0)       # nothing to do

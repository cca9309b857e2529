"""Softmax / LogSoftmax through the C-ABI against the CPU restatement of the reference's loops.  The kernel adds the
exponentials of a line as a tree, the reference one after the other, and the rounding of that sequential fp32 sum grows
with the length A of the axis: the outputs are held to max(1e-5, 16 sqrt(A) 2^-24) relative against the restatement, and
to 2e-6 relative against the float64 definition (which the tree sum follows more closely than the loop does)."""
import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import graph_runner as gr
from tests import util

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,axis", [((3,), 0), ((1, 3), 1), ((2, 3, 4), 1), ((2, 3, 4, 2), -2), ((64, 10), -1), ((7, 1000), 1), ((5, 129, 33), 1),
                                        ((3, 5, 70000), 2), ((300, 17), 0), ((4, 1), 1)])
@pytest.mark.parametrize("log", [False, True])
def test_softmax_matches_the_reference_loops(rt, shape, axis, log):
    X = (3 * util.normal(9201, int(np.prod(shape)))).reshape(shape)
    print("softmax", shape, axis, log, flush=True)
    got = gr.HipBackend(rt).softmax(X, axis, log)
    from scipy import special
    want = ob.softmax(X, axis, log)
    rel = max(1e-5, 16 * np.sqrt(X.shape[axis]) * 2.0 ** -24)
    if log:
        truth = special.log_softmax(X.astype(np.float64), axis=axis)
        assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 2 * rel)      # an error of the sum is an absolute error of its logarithm
        assert np.all(np.abs(got - truth) <= 1e-6 * np.abs(truth) + 2e-6)
    else:
        truth = special.softmax(X.astype(np.float64), axis=axis)
        assert np.all(np.abs(got - want) <= rel * want + 1e-30)
        assert np.all(np.abs(got - truth) <= 2e-6 * truth + 1e-30)
        assert np.allclose(got.sum(axis=axis), 1.0, atol=1e-5)


def test_softmax_extremes_and_errors(rt):
    be = gr.HipBackend(rt)
    big = np.array([[1000.0, 999.0, -1000.0], [-np.inf, 0.0, 0.0]], dtype=np.float32)
    got = be.softmax(big, 1, False)
    assert np.array_equal(got.view(np.uint32), ob.softmax(big, 1).view(np.uint32)) and got[1].tolist() == [0.0, 0.5, 0.5]
    x = util.to_dev(np.zeros(8, np.float32))
    with pytest.raises(R.SofieHipError, match="bad shape"):
        rt.call("sofie_hip_softmax_f32", util.ptr(x), util.ptr(x), 2, 0, 4, 0)
    with pytest.raises(R.SofieHipError, match="NULL"):
        rt.call("sofie_hip_softmax_f32", None, util.ptr(x), 2, 4, 1, 0)
    rt.call("sofie_hip_softmax_f32", None, None, 0, 4, 1, 0)      # an empty batch is no work

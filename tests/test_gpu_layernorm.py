"""LayerNormalization through the C-ABI against the CPU restatement of the reference's loops.  Mean and sum of squares are trees on
the device and loops in the reference: outputs are held to 2e-5 absolute + relative, the statistics to 1e-5 relative."""
import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import graph_runner as gr
from tests import util

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,axis", [((3, 4), -1), ((2, 3, 4, 5), 2), ((64, 768), 1), ((5, 7, 1000), 2), ((300, 3), 1), ((2, 4096), -1), ((6, 5, 4), 1)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_layernorm_matches_the_reference_loops(rt, shape, axis, with_bias):
    ax = axis + len(shape) if axis < 0 else axis
    n = int(np.prod(shape[ax:]))
    X = (2 * util.normal(9701, int(np.prod(shape))) + np.float32(0.5)).reshape(shape)
    scale = util.normal(9702, n).reshape(shape[ax:])
    bias = util.normal(9703, n).reshape(shape[ax:]) if with_bias else None
    print("layernorm", shape, axis, with_bias, flush=True)
    Y, mean, inv = gr.HipBackend(rt).layernorm(X, scale, bias, axis, 1e-5, stats=True)
    wY, wmean, winv = ob.layernorm(X, scale, bias, axis, 1e-5, stats=True)
    assert np.all(np.abs(Y - wY) <= 2e-5 * (1 + np.abs(wY)))
    assert np.allclose(mean, wmean, rtol=1e-5, atol=1e-6) and np.allclose(inv, winv, rtol=1e-5)
    assert wY.std() > 0.1


def test_layernorm_constant_row_and_errors(rt):
    be = gr.HipBackend(rt)
    Y, mean, inv = be.layernorm(np.full((2, 8), 3.0, np.float32), np.ones(8, np.float32), np.arange(8, dtype=np.float32), -1, 1e-4, stats=True)
    assert Y[1].tolist() == list(range(8)) and mean.tolist() == [3.0, 3.0] and np.allclose(inv, 100.0, rtol=1e-5)
    x = util.to_dev(np.zeros(8, np.float32))
    import ctypes as C
    with pytest.raises(R.SofieHipError, match="bad shape"):
        rt.call("sofie_hip_layernorm_f32", util.ptr(x), util.ptr(x), util.ptr(x), None, 2, 0, C.c_float(1e-5), None, None)
    with pytest.raises(R.SofieHipError, match="NULL"):
        rt.call("sofie_hip_layernorm_f32", util.ptr(x), util.ptr(x), None, None, 2, 4, C.c_float(1e-5), None, None)

"""The broadcasting binary operators and the pairwise steps of the n-ary ones through the C-ABI against the CPU restatement:
the bits of the IEEE operation for everything but Pow, which goes through the device's powf (held to 4 units in the last place)."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import graph_runner as gr
from tests import util

pytestmark = pytest.mark.gpu

SHAPES = [((5,), (5,)), ((2, 3, 4), (4,)), ((3, 1), (1, 4)), ((2, 1, 3, 1), (1, 1, 3, 4)), ((1,), (2, 3)), ((2, 3, 1, 5, 1, 2), (3, 4, 1, 7, 1)),
          ((1000, 513), (513,)), ((64, 1), (64, 300))]


@pytest.mark.parametrize("op", [R.BINARY_ADD, R.BINARY_SUB, R.BINARY_MUL, R.BINARY_DIV, R.BINARY_MAX, R.BINARY_MIN, R.BINARY_ADD_DIV])
def test_binary_operators_are_bit_exact(rt, op):
    be = gr.HipBackend(rt)
    for i, (sa, sb) in enumerate(SHAPES):
        A = util.normal(9300 + i, int(np.prod(sa)), 2.0).reshape(sa)
        B = util.normal(9400 + i, int(np.prod(sb)), 2.0).reshape(sb)
        print("binary", op, sa, sb, flush=True)
        got, want = be.binary(A, B, op, 3.0), ob.binary_broadcast(A, B, op, 3.0)
        assert got.shape == want.shape and np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_pow_and_special_values(rt):
    be = gr.HipBackend(rt)
    A = np.abs(util.normal(9501, 4000, 2.0)).reshape(40, 100) + np.float32(0.01)
    B = util.normal(9502, 100, 2.0)
    got, want = be.binary(A, B, R.BINARY_POW), ob.binary_broadcast(A, B, R.BINARY_POW)
    ulp = np.spacing(np.abs(want))
    assert np.all(np.abs(got.astype(np.float64) - want) <= 4 * ulp)
    # first-argument semantics of std::max / std::min with NaN and signed zeros; pow's special cases
    a = np.array([np.nan, 1.0, -0.0, 0.0, np.inf], np.float32)
    b = np.array([1.0, np.nan, 0.0, -0.0, -np.inf], np.float32)
    for op in (R.BINARY_MAX, R.BINARY_MIN, R.BINARY_DIV, R.BINARY_SUB):
        got, want = be.binary(a, b, op), ob.binary_broadcast(a, b, op)
        assert np.array_equal(np.isnan(got), np.isnan(want)), op
        ok = ~np.isnan(want)      # sign and payload of a NaN are not part of the operators' definition
        assert np.array_equal(got.view(np.uint32)[ok], want.view(np.uint32)[ok]), op
    p = be.binary(np.array([np.nan, 1.0, -8.0, -8.0, 0.0], np.float32), np.array([0.0, np.nan, 1.0 / 3, 2.0, -1.0], np.float32), R.BINARY_POW)
    assert p[0] == 1.0 and p[1] == 1.0 and np.isnan(p[2]) and p[3] == 64.0 and np.isposinf(p[4])


def test_binary_errors(rt):
    d = R.AddDesc()
    d.rank = 1
    d.y_shape[0], d.a_shape[0], d.b_shape[0] = 4, 4, 4
    x = util.to_dev(np.zeros(4, np.float32))
    d.A = d.B = d.Y = util.ptr(x)
    with pytest.raises(R.SofieHipError, match="unknown operator"):
        rt.call("sofie_hip_binary_f32", C.byref(d), 8, C.c_float(0))
    d.b_shape[0] = 3
    with pytest.raises(R.SofieHipError, match="cannot be broadcast"):
        rt.call("sofie_hip_binary_f32", C.byref(d), R.BINARY_MUL, C.c_float(0))

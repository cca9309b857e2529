"""Transpose and the pitched copy behind Concat through the C-ABI: pure data movement, so numpy's result is the definition and
the comparison is on the bits."""
import ctypes as C
import itertools

import numpy as np
import pytest

from sofie_amd import runtime as R
from tests import graph_runner as gr
from tests import util

pytestmark = pytest.mark.gpu


def test_transpose_every_permutation_up_to_rank_four_and_some_beyond(rt):
    be = gr.HipBackend(rt)
    for shape in [(7,), (3, 5), (2, 3, 4), (2, 3, 4, 5)]:
        X = util.normal(9600 + len(shape), int(np.prod(shape))).reshape(shape)
        for perm in itertools.permutations(range(len(shape))):
            got = be.transpose(X, list(perm))
            assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(np.transpose(X, perm)).view(np.uint32)), (shape, perm)
    X = util.normal(9610, 2 * 3 * 2 * 5 * 3 * 4).reshape(2, 3, 2, 5, 3, 4)
    for perm in [(5, 4, 3, 2, 1, 0), (0, 2, 1, 4, 3, 5), (3, 0, 5, 1, 4, 2)]:
        assert np.array_equal(be.transpose(X, list(perm)), np.transpose(X, perm))
    big = util.normal(9611, 1000 * 777).reshape(1000, 777)
    print("transpose 1000x777", flush=True)
    assert np.array_equal(be.transpose(big, [1, 0]), big.T)


def test_concat_along_every_axis(rt):
    be = gr.HipBackend(rt)
    base = (3, 4, 5)
    for axis in (0, 1, 2, -1):
        xs = []
        for i, n in enumerate((2, 1, 6)):
            shape = list(base)
            shape[axis] = n
            xs.append(util.normal(9620 + i, int(np.prod(shape))).reshape(shape))
        print("concat axis", axis, flush=True)
        assert np.array_equal(be.concat(xs, axis), np.concatenate(xs, axis=axis))


def test_shape_op_errors(rt):
    x = util.to_dev(np.zeros(24, np.float32))
    shape = (C.c_int64 * 6)(2, 3, 4, 1, 1, 1)
    with pytest.raises(R.SofieHipError, match="not a permutation"):
        rt.call("sofie_hip_transpose_f32", util.ptr(x), util.ptr(x), 3, shape, (C.c_int32 * 6)(0, 0, 2, 3, 4, 5))
    with pytest.raises(R.SofieHipError, match="rank"):
        rt.call("sofie_hip_transpose_f32", util.ptr(x), util.ptr(x), 7, shape, (C.c_int32 * 6)(0, 1, 2, 3, 4, 5))
    with pytest.raises(R.SofieHipError, match="multiples of 4"):
        rt.call("sofie_hip_copy_rows", util.ptr(x), C.c_size_t(8), util.ptr(x), C.c_size_t(8), C.c_size_t(2), C.c_size_t(6))
    with pytest.raises(R.SofieHipError, match="pitch"):
        rt.call("sofie_hip_copy_rows", util.ptr(x), C.c_size_t(4), util.ptr(x), C.c_size_t(8), C.c_size_t(2), C.c_size_t(8))

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


# ---- the strided read behind Slice, Split, Expand and Tile -------------------------------------------------------------------------------

def test_strided_gather_reproduces_numpy_views(rt):
    be = gr.HipBackend(rt)
    X = util.normal(9901, 7 * 9 * 11).reshape(7, 9, 11)
    views = [X[1:6:2, ::-1, 3:], X[::-3, 2:3, ::-4], X[:, :, 10:11], X[6:7], np.broadcast_to(X[:, 4:5, :], (7, 5, 11)), X.transpose(2, 0, 1), X[3, ::2, 1]]
    for v in views:
        print("strided gather", v.shape, v.strides, flush=True)
        assert np.array_equal(be.view(X, v), v)
    big = util.normal(9902, 300 * 1000).reshape(300, 1000)
    assert np.array_equal(be.view(big, big[::-1, ::-7]), big[::-1, ::-7])
    row = util.normal(9903, 5)
    assert np.array_equal(be.view(row, np.broadcast_to(row, (2000, 3, 5))), np.broadcast_to(row, (2000, 3, 5)))
    # Gather as the emitted code does it: one pitched copy per index
    assert np.array_equal(be.take(X, [[4, 0], [8, -1]], 1), np.take(X, [[4, 0], [8, -1]], axis=1))


def test_strided_gather_refuses_reads_outside_the_input(rt):
    import ctypes as C
    x = util.to_dev(np.zeros(24, np.float32))
    y = util.dev_empty((64,), np.float32)
    arr = lambda *v: (C.c_int64 * 6)(*(list(v) + [1] * (6 - len(v))))

    def call(rank, shape, strides, offset, n=24):
        rt.call("sofie_hip_strided_gather_f32", util.ptr(y), util.ptr(x), rank, shape, strides, offset, n)

    call(2, arr(4, 6), arr(6, 1), 0)                                    # the whole tensor
    call(2, arr(4, 6), arr(-6, -1), 23)                                 # backwards from its last element
    call(1, arr(0), arr(1000), 0)                                       # nothing to read
    with pytest.raises(R.SofieHipError, match=r"reads elements 1\.\.24 of an input of 24"):
        call(2, arr(4, 6), arr(6, 1), 1)
    with pytest.raises(R.SofieHipError, match=r"reads elements -1\.\.22"):
        call(2, arr(4, 6), arr(-6, -1), 22)
    with pytest.raises(R.SofieHipError, match="rank 7"):
        call(7, arr(1), arr(1), 0)
    with pytest.raises(R.SofieHipError, match="bad input size or offset"):
        call(1, arr(4), arr(1), -1)
    with pytest.raises(R.SofieHipError, match="NULL"):
        rt.call("sofie_hip_strided_gather_f32", None, util.ptr(x), 1, arr(4), arr(1), 0, 24)

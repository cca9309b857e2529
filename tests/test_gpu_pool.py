"""MaxPool / AveragePool through the C-ABI against the CPU restatement of the reference's generated loops.
The kernel adds the window in the loops' order, so the comparison is on the bits."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import graph_runner as gr
from tests import util

pytestmark = pytest.mark.gpu


def both(rt, X, mode, k, pads=None, strides=None, dilations=None, auto_pad="NOTSET", ceil_mode=0, include=0):
    axes = ob.pool_axes(X.shape[2:], k, pads, strides, dilations, auto_pad, ceil_mode)
    print("pool", mode, X.shape, "k", k, "pads", pads, "strides", strides, auto_pad, "ceil", ceil_mode, "include", include, flush=True)
    got = gr.hip_pool(rt, X, mode, axes, ceil_mode, include)
    want = ob.pool(X, mode, k, pads, strides, dilations, auto_pad, ceil_mode, include)
    return got, want


def same_bits(a, b):
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("mode", ["max", "average"])
def test_pool_sweep_of_geometries_is_bit_exact(rt, mode):
    rng = np.random.default_rng(21)
    for case in range(60):
        H, W = (int(v) for v in rng.integers(3, 20, 2))
        kh, kw = (int(v) for v in rng.integers(1, 5, 2))
        sh, sw = (int(v) for v in rng.integers(1, 4, 2))
        pads = [int(min(p, kk - 1)) for p, kk in zip(rng.integers(0, 3, 4), (kh, kw, kh, kw))]
        X = rng.standard_normal((int(rng.integers(1, 4)), int(rng.integers(1, 6)), H, W)).astype(np.float32)
        got, want = both(rt, X, mode, [kh, kw], pads, [sh, sw], None, "NOTSET", case % 2, (case // 2) % 2)
        assert same_bits(got, want), case


@pytest.mark.parametrize("mode", ["max", "average"])
@pytest.mark.parametrize("auto_pad", ["SAME_UPPER", "SAME_LOWER", "VALID"])
def test_pool_auto_pad_and_one_dimension(rt, mode, auto_pad):
    X = util.normal(9101, 3 * 5 * 37).reshape(3, 5, 37)
    got, want = both(rt, X, mode, [4], None, [3], None, auto_pad)
    assert same_bits(got, want)
    X2 = util.normal(9102, 2 * 3 * 11 * 14).reshape(2, 3, 11, 14)
    got, want = both(rt, X2, mode, [3, 2], None, [2, 3], None, auto_pad)
    assert same_bits(got, want)


@pytest.mark.parametrize("mode", ["max", "average"])
def test_pool_over_three_axes_is_bit_exact(rt, mode):
    """Volumes [N, C, D, H, W]: every axis with its own extent, window, stride and padding, both divisor conventions, ceil_mode."""
    rng = np.random.default_rng(23)
    for case in range(40):
        sp = [int(v) for v in rng.integers(2, 11, 3)]
        k = [int(min(v, n)) for v, n in zip(rng.integers(1, 4, 3), sp)]
        st = [int(v) for v in rng.integers(1, 4, 3)]
        pads = [int(min(p, kk - 1)) for p, kk in zip(rng.integers(0, 3, 6), k + k)]
        X = rng.standard_normal((int(rng.integers(1, 3)), int(rng.integers(1, 5)), *sp)).astype(np.float32)
        got, want = both(rt, X, mode, k, pads, st, None, "NOTSET", case % 2, (case // 2) % 2)
        assert same_bits(got, want), case
    X = util.normal(9104, 2 * 8 * 16 * 40 * 40).reshape(2, 8, 16, 40, 40)
    got, want = both(rt, X, mode, [2, 3, 3], [0, 1, 1, 0, 1, 1], [2, 2, 2])
    assert got.shape == (2, 8, 8, 20, 20) and same_bits(got, want)


def test_pool_at_the_size_of_a_network_stem(rt):
    """64 x 64 planes of 112 x 112 -> MaxPool 3x3 / 2 / pad 1 -> 56 x 56: more outputs than one pass of the grid covers."""
    X = util.normal(9103, 64 * 64 * 112 * 112).reshape(64, 64, 112, 112)
    got, want = both(rt, X, "max", [3, 3], [1, 1, 1, 1], [2, 2])
    assert got.shape == (64, 64, 56, 56) and same_bits(got, want)
    got, want = both(rt, X[:8], "average", [7, 7], [3, 3, 3, 3], [4, 4], include=1)
    assert same_bits(got, want)


def test_pool_special_values_and_dilated_window(rt):
    X = util.normal(9104, 2 * 2 * 9 * 9).reshape(2, 2, 9, 9).copy()
    X[0, 0, :4, :4] = np.nan
    X[1, 1, 2, 3] = np.inf
    X[1, 0, 5, 5] = -np.inf
    got, want = both(rt, X, "max", [2, 2], None, [2, 2])
    assert same_bits(got, want) and np.isneginf(got[0, 0, 0, 0])      # a window of NaNs only keeps the starting value
    got, want = both(rt, X, "average", [3, 3], [1, 1, 1, 1], [1, 1])
    assert same_bits(got, want)
    got, want = both(rt, X, "max", [2, 2], None, [1, 1], [2, 2])    # the reference's dense window of the dilated extent
    assert got.shape == (2, 2, 7, 7) and same_bits(got, want)


def test_pool_empty_and_errors(rt):
    x = util.to_dev(np.zeros(64, np.float32))
    y = util.to_dev(np.full(64, 7.0, np.float32))

    def desc(**kw):
        base = dict(planes=1, H=8, W=8, OH=7, OW=7, kh=2, kw=2, pad_h0=0, pad_w0=0, pad_h1=0, pad_w1=0, stride_h=1, stride_w=1, mode=R.POOL_MAX,
                    count_include_pad=0, dynamic_divisor=0)
        base.update(kw)
        return R.PoolDesc(**base)
    rt.call("sofie_hip_pool_f32", C.byref(desc(planes=0)), util.ptr(y), util.ptr(x))      # no planes: nothing is written
    rt.sync()
    assert np.all(util.to_host(y) == 7.0)
    with pytest.raises(R.SofieHipError, match="unknown mode"):
        rt.call("sofie_hip_pool_f32", C.byref(desc(mode=5)), util.ptr(y), util.ptr(x))
    with pytest.raises(R.SofieHipError, match="does not fit"):
        rt.call("sofie_hip_pool_f32", C.byref(desc(OH=9)), util.ptr(y), util.ptr(x))
    with pytest.raises(R.SofieHipError, match="bad stride"):
        rt.call("sofie_hip_pool_f32", C.byref(desc(stride_w=0)), util.ptr(y), util.ptr(x))
    with pytest.raises(R.SofieHipError, match="NULL"):
        rt.call("sofie_hip_pool_f32", C.byref(desc()), None, util.ptr(x))

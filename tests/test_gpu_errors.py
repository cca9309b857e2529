"""Error behaviour of the C-ABI: a bad argument is a non-zero status with a message that names the function and the
argument (the emitted Session turns it into std::runtime_error, the reference's convention), and never a launch."""
import ctypes as C

import numpy as np
import pytest

from sofie_amd import SofieHipError, runtime as R
from tests import util

pytestmark = pytest.mark.gpu


def test_gemm_f32_argument_checks(rt):
    A, B, Y = util.to_dev(np.zeros((4, 3), np.float32)), util.to_dev(np.zeros((3, 5), np.float32)), util.dev_empty((4, 5), np.float32)
    d = R.GemmF32Desc()
    d.M, d.N, d.K, d.alpha, d.beta, d.batch = 4, 5, 3, 1.0, 1.0, 1
    d.A, d.B, d.Y = util.ptr(A), util.ptr(B), util.ptr(Y)
    rt.call("sofie_hip_gemm_f32", C.byref(d))        # the valid call
    d.bias_mode = R.BIAS_ROW                            # bias mode without a bias tensor
    with pytest.raises(SofieHipError, match="bias mode set but C is NULL"):
        rt.call("sofie_hip_gemm_f32", C.byref(d))
    d.bias_mode, d.lda = R.BIAS_NONE, 2                 # leading dimension smaller than K
    with pytest.raises(SofieHipError, match="leading dimension too small"):
        rt.call("sofie_hip_gemm_f32", C.byref(d))
    d.lda, d.act = 0, 99
    with pytest.raises(SofieHipError, match="unknown activation"):
        rt.call("sofie_hip_gemm_f32", C.byref(d))
    d.act, d.M = 0, -1
    with pytest.raises(SofieHipError, match="negative dimension"):
        rt.call("sofie_hip_gemm_f32", C.byref(d))
    d.M, d.batch = 4, 0
    with pytest.raises(SofieHipError, match="batch must be >= 1"):
        rt.call("sofie_hip_gemm_f32", C.byref(d))
    rt.sync()


def test_conv_argument_checks(rt):
    d = R.ConvDesc()
    d.N, d.C, d.H, d.W, d.Cout, d.kh, d.kw = 1, 4, 6, 6, 6, 3, 3
    d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
    d.group, d.OH, d.OW = 1, 4, 4
    X, W, Y = util.to_dev(np.zeros((1, 4, 6, 6), np.float32)), util.to_dev(np.zeros((6, 4, 3, 3), np.float32)), util.dev_empty((1, 6, 4, 4), np.float32)
    rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(X), util.ptr(W), None, 0, C.c_float(0), util.ptr(Y), None, None)
    d.OH = 5                                            # the caller's shape inference disagrees
    with pytest.raises(SofieHipError, match="does not match the descriptor"):
        rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(X), util.ptr(W), None, 0, C.c_float(0), util.ptr(Y), None, None)
    d.OH, d.group = 4, 3                                # groups that do not divide the channels
    with pytest.raises(SofieHipError, match="does not divide"):
        rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(X), util.ptr(W), None, 0, C.c_float(0), util.ptr(Y), None, None)
    d.group, d.kh = 1, 9                                # kernel larger than the padded image
    with pytest.raises(SofieHipError, match="larger than the padded image"):
        rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(X), util.ptr(W), None, 0, C.c_float(0), util.ptr(Y), None, None)
    d.kh = 3
    a = R.ConvI8Args()
    a.X, a.W, a.Y, a.out = util.ptr(X), util.ptr(W), util.ptr(Y), R.I8OUT_I8   # int8 output without a scale
    with pytest.raises(SofieHipError, match="scale is NULL"):
        rt.call("sofie_hip_conv_i8", C.byref(d), C.byref(a))
    rt.sync()


def test_elementwise_and_arena_argument_checks(rt):
    x = util.to_dev(np.ones(8, np.float32))
    q = util.dev_empty((8,), np.int8)
    with pytest.raises(SofieHipError, match="scale must be positive"):
        rt.call("sofie_hip_quantize_linear", util.ptr(q), util.ptr(x), C.c_size_t(8), C.c_float(0.0))
    with pytest.raises(SofieHipError, match="NULL pointer"):
        rt.call("sofie_hip_quantize_linear", None, util.ptr(x), C.c_size_t(8), C.c_float(1.0))
    rt.call("sofie_hip_quantize_linear", None, None, C.c_size_t(0), C.c_float(1.0))       # empty tensors are no-ops
    with pytest.raises(SofieHipError, match="bad shape"):
        rt.call("sofie_hip_batchnorm_f32", util.ptr(x), util.ptr(x), util.ptr(x), util.ptr(x), util.ptr(x), 1, 0, 8, 0)
    from sofie_amd import Runtime
    own = Runtime(0)
    try:
        with pytest.raises(SofieHipError, match="power of two"):
            own.call("sofie_hip_arena_create", C.c_size_t(1024), C.c_size_t(100))
        own.call("sofie_hip_arena_create", C.c_size_t(1024), C.c_size_t(256))
        with pytest.raises(SofieHipError, match="already has an arena"):
            own.call("sofie_hip_arena_create", C.c_size_t(1024), C.c_size_t(256))
        assert own.lib.sofie_hip_arena_ptr(own.ctx, C.c_size_t(4096)) is None          # beyond the arena
    finally:
        own.close()
    rt.sync()

"""fp32 Gemm / Conv / elementwise operators through the C-ABI against the CPU restatement of SOFIE's
generated code.  Tolerance: |got - want| <= 1e-5 * (|want| + sum_k |a_k b_k|) -- 1e-5 relative to the
magnitude the dot product is formed from (the summation order of a GEMM is not part of its definition)."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import util

pytestmark = pytest.mark.gpu


def gemm(rt, A, B, Cb, M, N, K, transA=0, transB=0, alpha=1.0, beta=1.0, bias_mode=0, act=0, act_alpha=0.0, batch=1,
         strides=(0, 0, 0, 0)):
    dA, dB = util.to_dev(A), util.to_dev(B)
    dC = None if Cb is None else util.to_dev(Cb)
    dY = util.dev_empty((batch, M, N), np.float32)
    d = R.GemmF32Desc()
    d.M, d.N, d.K, d.transA, d.transB = M, N, K, transA, transB
    d.alpha, d.beta = alpha, beta
    d.A, d.B, d.C, d.Y = util.ptr(dA), util.ptr(dB), util.ptr(dC), util.ptr(dY)
    d.bias_mode, d.act, d.act_alpha = bias_mode, act, act_alpha
    d.batch = batch
    d.strideA, d.strideB, d.strideC, d.strideY = strides
    import torch
    torch.cuda.synchronize()
    print("gemm_f32 M=%d N=%d K=%d tA=%d tB=%d bias=%d act=%d batch=%d" % (M, N, K, transA, transB, bias_mode, act, batch), flush=True)
    rt.call("sofie_hip_gemm_f32", C.byref(d))
    rt.sync()
    y = util.to_host(dY)
    return y[0] if batch == 1 else y


def close(got, want, mag, rel=1e-5):
    return np.all(np.abs(got.astype(np.float64) - want) <= rel * (np.abs(want) + mag) + 1e-30)


@pytest.mark.parametrize("M,N,K,transA,transB", [(64, 128, 784, 0, 1), (64, 64, 128, 0, 1), (64, 10, 64, 0, 1), (16, 50, 100, 0, 0),
                                                 (7, 5, 3, 1, 0), (65, 67, 33, 1, 1), (1, 1, 1, 0, 0), (130, 70, 257, 0, 0), (9, 17, 520, 0, 1), (12, 20, 600, 1, 0)])
@pytest.mark.parametrize("bias_mode,act", [(0, 0), (1, 1), (2, 0), (3, 2), (4, 3), (1, 4)])
@pytest.mark.parametrize("kernel", ["tiles64", "wave8x8"])
def test_gemm_f32_matches_sofie_cpu_semantics(rt, M, N, K, transA, transB, bias_mode, act, kernel, opt):
    # both fp32 kernels on every shape: the 64x64-tile one and the one-wave 8x8-tile one for small products
    opt("f32_skinny", 1 if kernel == "wave8x8" else 0)
    A = util.normal(1, M * K).reshape((K, M) if transA else (M, K))
    B = util.normal(2, N * K, 0.05).reshape((N, K) if transB else (K, N))
    Cshape = {0: None, 1: (N,), 2: (M, 1), 3: (1,), 4: (M, N)}[bias_mode]
    Cb = None if Cshape is None else util.normal(3, int(np.prod(Cshape))).reshape(Cshape)
    alpha, beta = 1.25, 0.5
    got = gemm(rt, A, B, Cb, M, N, K, transA, transB, alpha, beta, bias_mode, act, 0.1)
    want = ob.gemm_f32(A, B, Cb, M=M, N=N, K=K, transA=transA, transB=transB, alpha=alpha, beta=beta, bias_mode=bias_mode,
                       act=act, act_alpha=0.1)
    opA = A.T if transA else A
    opB = B.T if transB else B
    mag = np.abs(alpha) * (np.abs(opA).astype(np.float64) @ np.abs(opB).astype(np.float64)) + 1.0
    assert close(got, want.astype(np.float64), mag)
    # float64 textbook arbiter for the linear part
    if act == 0:
        ref = alpha * (opA.astype(np.float64) @ opB.astype(np.float64))
        if bias_mode in (1, 2, 3):
            ref = ref + Cb.astype(np.float64)
        elif bias_mode == 4:
            ref = ref + beta * Cb.astype(np.float64)
        assert close(got, ref, mag)


def test_relu_edge_cases_follow_the_cpu_helper(rt):
    # Relu(NaN) = 0 and Relu(-0) = +0 on SOFIE's CPU path
    x = np.array([np.nan, -0.0, 0.0, -1.0, 2.5, np.inf, -np.inf], dtype=np.float32)
    dx = util.to_dev(x)
    dy = util.dev_empty(x.shape, np.float32)
    rt.call("sofie_hip_unary_f32", util.ptr(dy), util.ptr(dx), C.c_size_t(x.size), R.ACT_RELU, C.c_float(0))
    rt.sync()
    got = util.to_host(dy)
    want = ob.unary(x, R.ACT_RELU)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_stacked_matmul(rt):
    b, M, N, K = 5, 12, 9, 20
    A = util.normal(5, b * M * K).reshape(b, M, K)
    B = util.normal(6, b * K * N).reshape(b, K, N)
    got = gemm(rt, A, B, None, M, N, K, batch=b, strides=(M * K, K * N, 0, M * N))
    want = np.einsum("bmk,bkn->bmn", A.astype(np.float64), B.astype(np.float64))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # shared B (stride 0)
    got = gemm(rt, A, B[0], None, M, N, K, batch=b, strides=(M * K, 0, 0, M * N))
    want = np.einsum("bmk,kn->bmn", A.astype(np.float64), B[0].astype(np.float64))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("act", [R.ACT_RELU, R.ACT_LEAKYRELU, R.ACT_SIGMOID, R.ACT_GELU, R.ACT_GELU_TANH, R.ACT_TANH])
@pytest.mark.parametrize("n", [1, 7, 4096 + 3])
def test_unary(rt, act, n):
    x = util.normal(10 + act, n, 2.0)
    dx = util.to_dev(x)
    dy = util.dev_empty((n,), np.float32)
    rt.call("sofie_hip_unary_f32", util.ptr(dy), util.ptr(dx), C.c_size_t(n), act, C.c_float(0.2))
    rt.sync()
    want = ob.unary(x, act, 0.2)
    assert np.allclose(util.to_host(dy), want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("ash,bsh", [((4, 5), (4, 5)), ((4, 5), (5,)), ((4, 1), (1, 5)), ((2, 3, 4, 5), (3, 1, 5)), ((1,), (6, 7))])
def test_add_broadcast(rt, ash, bsh):
    A = util.normal(20, int(np.prod(ash))).reshape(ash)
    B = util.normal(21, int(np.prod(bsh))).reshape(bsh)
    ysh = np.broadcast_shapes(ash, bsh)
    rank = len(ysh)
    d = R.AddDesc()
    d.rank = rank
    for i, v in enumerate(ysh):
        d.y_shape[i] = v
    for i, v in enumerate((1,) * (rank - len(ash)) + tuple(ash)):
        d.a_shape[i] = v
    for i, v in enumerate((1,) * (rank - len(bsh)) + tuple(bsh)):
        d.b_shape[i] = v
    dA, dB = util.to_dev(A), util.to_dev(B)
    dY = util.dev_empty(ysh, np.float32)
    d.A, d.B, d.Y = util.ptr(dA), util.ptr(dB), util.ptr(dY)
    rt.call("sofie_hip_add_f32", C.byref(d))
    rt.sync()
    got = util.to_host(dY)
    assert np.array_equal(got, A + B)
    assert np.array_equal(got, ob.add_broadcast(A, B))


def conv_desc(N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group):
    OH, OW = ob.conv_out_hw(H, W, kh, kw, pads, strides, dils)
    d = R.ConvDesc()
    (d.N, d.C, d.H, d.W, d.Cout, d.kh, d.kw) = (N, Cc, H, W, Cout, kh, kw)
    (d.pad_h0, d.pad_w0, d.pad_h1, d.pad_w1) = pads
    (d.stride_h, d.stride_w), (d.dil_h, d.dil_w) = strides, dils
    d.group, d.OH, d.OW = group, OH, OW
    return d


CONV_CASES = [
    # N, C, H, W, Cout, kh, kw, pads, strides, dils, group
    (1, 1, 5, 5, 1, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),
    (2, 3, 9, 7, 5, 3, 3, (0, 0, 0, 0), (1, 1), (1, 1), 1),
    (2, 4, 8, 8, 6, 3, 2, (1, 0, 2, 1), (2, 1), (1, 1), 2),
    (1, 2, 10, 10, 4, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2), 1),
    (3, 8, 6, 6, 8, 1, 1, (0, 0, 0, 0), (1, 1), (1, 1), 4),
    (2, 3, 1, 20, 4, 1, 5, (0, 2, 0, 2), (1, 2), (1, 1), 1),
    (4, 3, 16, 16, 64, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("with_bias,act", [(False, 0), (True, 1)])
def test_conv_f32(rt, case, with_bias, act):
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.uniform01(30, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.normal(31, Cout * (Cc // group) * kh * kw, 0.3).reshape(Cout, Cc // group, kh, kw)
    b = util.normal(32, Cout) if with_bias else None
    d = conv_desc(N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group)
    dX, dW = util.to_dev(X), util.to_dev(Wt)
    db = None if b is None else util.to_dev(b)
    dY = util.dev_empty((N, Cout, d.OH, d.OW), np.float32)
    print("conv_f32", case, flush=True)
    rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(dX), util.ptr(dW), util.ptr(db), act, C.c_float(0), util.ptr(dY), None, None)
    rt.sync()
    want = ob.conv_f32(X, Wt, b, pads=pads, strides=strides, dils=dils, group=group, act=act)
    assert np.allclose(util.to_host(dY), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("case", [
    # N, C, (D,H,W), Cout, (kd,kh,kw), pads {d0,h0,w0,d1,h1,w1}, strides, dils, group
    (1, 1, (3, 4, 4), 2, (2, 3, 3), (0, 1, 1, 0, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    (2, 4, (5, 6, 7), 6, (3, 2, 3), (1, 0, 2, 0, 1, 1), (2, 1, 2), (1, 1, 1), 2),
    (1, 2, (7, 5, 6), 3, (2, 3, 2), (2, 1, 0, 1, 2, 1), (1, 2, 1), (2, 1, 2), 1),
    (1, 6, (4, 4, 4), 6, (3, 3, 3), (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), 3),
    (2, 8, (8, 12, 10), 40, (3, 3, 3), (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    (1, 3, (2, 3, 3), 2, (1, 1, 1), (0, 0, 0, 0, 0, 0), (1, 1, 1), (1, 1, 1), 1),
])
@pytest.mark.parametrize("with_bias,act", [(False, 0), (True, 1)])
def test_conv3d_f32(rt, case, with_bias, act):
    """3-D convolution: the im2col-3D + Gemm of the reference's CPU operator, restated in the oracle, against the kernel that
    gathers the taps while it loads its tiles."""
    N, Cc, sp, Cout, k, pads, strides, dils, group = case
    X = util.uniform01(33, N * Cc * int(np.prod(sp))).reshape(N, Cc, *sp)
    Wt = util.normal(34, Cout * (Cc // group) * int(np.prod(k)), 0.3).reshape(Cout, Cc // group, *k)
    b = util.normal(35, Cout) if with_bias else None
    out = [(sp[a] + pads[a] + pads[a + 3] - (dils[a] * (k[a] - 1) + 1)) // strides[a] + 1 for a in range(3)]
    d = R.Conv3dDesc()
    (d.N, d.C, d.D, d.H, d.W, d.Cout, d.kd, d.kh, d.kw) = (N, Cc, *sp, Cout, *k)
    d.pad, d.stride, d.dil = (C.c_int32 * 6)(*pads), (C.c_int32 * 3)(*strides), (C.c_int32 * 3)(*dils)
    d.group, d.OD, d.OH, d.OW = group, *out
    dX, dW = util.to_dev(X), util.to_dev(Wt)
    db = None if b is None else util.to_dev(b)
    dY = util.dev_empty((N, Cout, *out), np.float32)
    print("conv3d_f32", case, flush=True)
    rt.call("sofie_hip_conv3d_f32", C.byref(d), util.ptr(dX), util.ptr(dW), util.ptr(db), act, C.c_float(0), util.ptr(dY), None, None)
    rt.sync()
    want = ob.conv3d_f32(X, Wt, b, pads=pads, strides=strides, dils=dils, group=group, act=act)
    assert want.shape == (N, Cout, *out)
    assert np.allclose(util.to_host(dY), want, rtol=1e-5, atol=1e-5)


def test_conv3d_refuses_inconsistent_geometry(rt):
    d = R.Conv3dDesc()
    (d.N, d.C, d.D, d.H, d.W, d.Cout, d.kd, d.kh, d.kw) = (1, 2, 4, 4, 4, 2, 3, 3, 3)
    d.pad, d.stride, d.dil = (C.c_int32 * 6)(*[0] * 6), (C.c_int32 * 3)(1, 1, 1), (C.c_int32 * 3)(1, 1, 1)
    d.group, d.OD, d.OH, d.OW = 1, 2, 2, 3  # OW should be 2
    x = util.to_dev(np.zeros(2 * 64, np.float32))
    w = util.to_dev(np.zeros(2 * 2 * 27, np.float32))
    y = util.dev_empty((2 * 12,), np.float32)
    with pytest.raises(R.SofieHipError):
        rt.call("sofie_hip_conv3d_f32", C.byref(d), util.ptr(x), util.ptr(w), None, 0, C.c_float(0), util.ptr(y), None, None)
    d.OW, d.group = 2, 3  # 2 channels do not split into 3 groups
    with pytest.raises(R.SofieHipError):
        rt.call("sofie_hip_conv3d_f32", C.byref(d), util.ptr(x), util.ptr(w), None, 0, C.c_float(0), util.ptr(y), None, None)


def test_global_avg_pool(rt):
    X = util.normal(40, 3 * 7 * 33).reshape(3, 7, 33)
    dX = util.to_dev(X)
    dY = util.dev_empty((21,), np.float32)
    rt.call("sofie_hip_global_avg_pool_f32", util.ptr(dY), util.ptr(dX), 21, 33)
    rt.sync()
    want = ob.global_avg_pool(X.reshape(3, 7, 33, 1)).reshape(21)
    assert np.allclose(util.to_host(dY), want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(4, 6), (3, 5, 7), (2, 8, 5, 6), (1, 1, 1, 1)])
@pytest.mark.parametrize("relu", [0, 1])
def test_batchnorm_same_three_roundings_as_the_cpu_loop(rt, shape, relu):
    Cc = shape[1]
    X = util.normal(90, int(np.prod(shape))).reshape(shape)
    gamma, beta = (0.5 + util.uniform01(91, Cc)).astype(np.float32), util.normal(92, Cc)
    mean, var = util.normal(93, Cc, 0.3), (0.1 + util.uniform01(94, Cc)).astype(np.float32)
    want, fused = ob.batchnorm(X, gamma, beta, mean, var, eps=1e-5, relu=relu)
    dX, dF, dM, dB = util.to_dev(X), util.to_dev(fused), util.to_dev(mean), util.to_dev(beta)
    dY = util.dev_empty(shape, np.float32)
    import torch
    torch.cuda.synchronize()
    rt.call("sofie_hip_batchnorm_f32", util.ptr(dY), util.ptr(dX), util.ptr(dF), util.ptr(dM), util.ptr(dB), shape[0], Cc,
            int(np.prod(shape[2:])), relu)
    rt.sync()
    assert np.array_equal(util.to_host(dY).view(np.uint32), want.view(np.uint32))


# ---- the other one-to-one operators and chains of them -------------------------------------------------------

def unary_domain(code, n, seed):
    """Inputs inside each operator's domain, away from its singularities."""
    u = util.uniform01(seed, n)
    z = util.normal(seed + 1, n, 2.0)
    return {R.ACT_RECIPROCAL: np.where(z >= 0, 0.1 + np.abs(z), -0.1 - np.abs(z)), R.ACT_SQRT: u * 9, R.ACT_LOG: 0.01 + u * 50,
            R.ACT_ACOSH: 1 + u * 20, R.ACT_ATANH: (u - 0.5) * 1.9, R.ACT_EXP: z * 1.5, R.ACT_SOFTPLUS: z * 12}.get(code, z).astype(np.float32)


BASIC_UNARY = [R.ACT_RECIPROCAL, R.ACT_SQRT, R.ACT_NEG, R.ACT_EXP, R.ACT_LOG, R.ACT_SIN, R.ACT_COS, R.ACT_ABS, R.ACT_SOFTPLUS, R.ACT_ATAN,
               R.ACT_FLOOR, R.ACT_ASINH, R.ACT_ACOSH, R.ACT_ATANH]


@pytest.mark.parametrize("code", BASIC_UNARY)
@pytest.mark.parametrize("n", [5, 4096 + 3])
def test_basic_unary_operators(rt, code, n):
    x = unary_domain(code, n, 300 + code)
    dx = util.to_dev(x)
    dy = util.dev_empty((n,), np.float32)
    rt.call("sofie_hip_unary_f32", util.ptr(dy), util.ptr(dx), C.c_size_t(n), code, C.c_float(0))
    rt.sync()
    want = ob.unary(x, code, 0.0)
    got = util.to_host(dy)
    assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(1.0, np.abs(want)))
    if code in (R.ACT_NEG, R.ACT_ABS, R.ACT_FLOOR, R.ACT_SQRT, R.ACT_RECIPROCAL):     # correctly rounded on both sides
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def run_chain(rt, x, ops):
    dx = util.to_dev(x)
    dy = util.dev_empty(x.shape, np.float32)
    rt.call("sofie_hip_unary_chain_f32", util.ptr(dy), util.ptr(dx), C.c_size_t(x.size), C.byref(R.PostOps.of(ops)))
    rt.sync()
    return util.to_host(dy)


def test_unary_chain_is_the_composition(rt):
    x = util.normal(400, 1000 + 3, 2.0)
    ops = [(R.ACT_LEAKYRELU, 0.1, 0.0), (R.ACT_EXP, 0.0, 0.0), (R.ACT_CLIP, 0.5, 3.0), (R.ACT_LOG, 0.0, 0.0)]
    got = run_chain(rt, x, ops)
    want = ob.unary_chain(x, ops)
    assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(1.0, np.abs(want)))
    assert want.min() >= np.log(np.float32(0.5)) - 1e-6 and want.max() <= np.log(np.float32(3.0)) + 1e-6
    # Clip alone is exact, bounds included; an empty chain and a chain of NONE copy
    clip = run_chain(rt, x, [(R.ACT_CLIP, -0.25, 0.75)])
    assert np.array_equal(clip, np.maximum(np.float32(-0.25), np.minimum(np.float32(0.75), x)))
    assert np.array_equal(run_chain(rt, x, []), x) and np.array_equal(run_chain(rt, x, [(R.ACT_NONE, 0, 0)] * 4), x)


def test_chain_errors(rt):
    x = util.to_dev(np.zeros(8, np.float32))
    bad = R.PostOps.of([(R.ACT_RELU, 0, 0)])
    bad.count = 5
    with pytest.raises(R.SofieHipError, match="more than 4"):
        rt.call("sofie_hip_unary_chain_f32", util.ptr(x), util.ptr(x), C.c_size_t(8), C.byref(bad))
    with pytest.raises(R.SofieHipError, match="unknown operator 99"):
        rt.call("sofie_hip_unary_chain_f32", util.ptr(x), util.ptr(x), C.c_size_t(8), C.byref(R.PostOps.of([(99, 0, 0)])))
    with pytest.raises(R.SofieHipError, match="NULL"):
        rt.call("sofie_hip_unary_chain_f32", util.ptr(x), util.ptr(x), C.c_size_t(8), None)


@pytest.mark.parametrize("kernel", ["tiles64", "wave8x8"])
@pytest.mark.parametrize("M,N,K", [(6, 12, 20), (70, 33, 129)])
def test_gemm_with_a_chain_in_its_store(rt, M, N, K, kernel, opt):
    opt("f32_skinny", 1 if kernel == "wave8x8" else 0)
    A = util.normal(410, M * K).reshape(M, K)
    B = util.normal(411, K * N, 0.1).reshape(K, N)
    bias = util.normal(412, N)
    ops = [(R.ACT_SIGMOID, 0, 0), (R.ACT_TANH, 0, 0), (R.ACT_CLIP, 0.2, 0.6), (R.ACT_SQRT, 0, 0)]
    dA, dB, dC = util.to_dev(A), util.to_dev(B), util.to_dev(bias)
    dY = util.dev_empty((M, N), np.float32)
    post = R.PostOps.of(ops)
    d = R.GemmF32Desc()
    d.M, d.N, d.K, d.alpha, d.beta, d.batch = M, N, K, 1.0, 1.0, 1
    d.A, d.B, d.C, d.Y = util.ptr(dA), util.ptr(dB), util.ptr(dC), util.ptr(dY)
    d.bias_mode, d.act, d.act_alpha = R.BIAS_ROW, R.ACT_LEAKYRELU, 0.1
    d.post = C.pointer(post)
    print("gemm_f32 with post ops", M, N, K, kernel, flush=True)
    rt.call("sofie_hip_gemm_f32", C.byref(d))
    rt.sync()
    lin = ob.gemm_f32(A, B, bias, M=M, N=N, K=K, bias_mode=1, act=R.ACT_LEAKYRELU, act_alpha=0.1)
    want = ob.unary_chain(lin, ops)
    got = util.to_host(dY)
    # the chain is a contraction here (sigmoid, tanh), so the GEMM's summation-order freedom stays below 1e-5 absolute
    assert np.abs(got - want).max() <= 1e-5 and want.std() > 0.01


def test_conv_with_a_chain_in_its_store(rt):
    N, Cc, H, W, Cout = 2, 3, 9, 7, 5
    X = util.uniform01(420, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.normal(421, Cout * Cc * 9, 0.3).reshape(Cout, Cc, 3, 3)
    b = util.normal(422, Cout)
    ops = [(R.ACT_ABS, 0, 0), (R.ACT_SOFTPLUS, 0, 0), (R.ACT_RECIPROCAL, 0, 0)]
    d = conv_desc(N, Cc, H, W, Cout, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1)
    dX, dW, db = util.to_dev(X), util.to_dev(Wt), util.to_dev(b)
    dY = util.dev_empty((N, Cout, d.OH, d.OW), np.float32)
    post = R.PostOps.of(ops)
    rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(dX), util.ptr(dW), util.ptr(db), R.ACT_TANH, C.c_float(0), util.ptr(dY), C.byref(post), None)
    rt.sync()
    want = ob.unary_chain(ob.conv_f32(X, Wt, b, pads=(1, 1, 1, 1), strides=(1, 1), dils=(1, 1), group=1, act=R.ACT_TANH), ops)
    assert np.abs(util.to_host(dY) - want).max() <= 1e-5 and want.std() > 0.01


@pytest.mark.parametrize("kernel", ["tiles64", "wave8x8"])
@pytest.mark.parametrize("M,N,K,batch", [(6, 12, 20, 1), (70, 33, 129, 1), (9, 10, 16, 3)])
def test_gemm_with_a_residual_operand(rt, M, N, K, batch, kernel, opt):
    """Y = act(alpha A B + bias + R): the Add of a same-shaped tensor behind the product, inside the store, before the activation."""
    opt("f32_skinny", 1 if kernel == "wave8x8" else 0)
    A = util.normal(430, batch * M * K).reshape(batch, M, K)
    B = util.normal(431, K * N, 0.1).reshape(K, N)
    bias = util.normal(432, N)
    Rr = util.normal(433, batch * M * N).reshape(batch, M, N)
    dA, dB, dC, dR = util.to_dev(A), util.to_dev(B), util.to_dev(bias), util.to_dev(Rr)
    dY = util.dev_empty((batch, M, N), np.float32)
    d = R.GemmF32Desc()
    d.M, d.N, d.K, d.alpha, d.beta, d.batch = M, N, K, 1.0, 1.0, batch
    d.strideA, d.strideB, d.strideC, d.strideY = M * K, 0, 0, M * N
    d.A, d.B, d.C, d.Y, d.residual = util.ptr(dA), util.ptr(dB), util.ptr(dC), util.ptr(dY), util.ptr(dR)
    d.bias_mode, d.act = R.BIAS_ROW, R.ACT_RELU
    print("gemm_f32 with residual", M, N, K, batch, kernel, flush=True)
    rt.call("sofie_hip_gemm_f32", C.byref(d))
    rt.sync()
    got = util.to_host(dY)
    for b in range(batch):
        lin = ob.gemm_f32(A[b], B, bias, M=M, N=N, K=K, bias_mode=1, act=0)
        want = ob.unary(ob.add_broadcast(lin, Rr[b]), R.ACT_RELU, 0.0)
        mag = np.abs(A[b]).astype(np.float64) @ np.abs(B).astype(np.float64) + 1.0
        assert close(got[b], want.astype(np.float64), mag)
    assert (got > 0).any() and (got == 0).any()


def test_conv_with_a_residual_operand(rt):
    N, Cc, H, W, Cout = 2, 8, 6, 6, 8
    X = util.normal(440, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.normal(441, Cout * Cc * 9, 0.15).reshape(Cout, Cc, 3, 3)
    b = util.normal(442, Cout)
    d = conv_desc(N, Cc, H, W, Cout, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1)
    dX, dW, db = util.to_dev(X), util.to_dev(Wt), util.to_dev(b)
    dY = util.dev_empty((N, Cout, d.OH, d.OW), np.float32)
    rt.call("sofie_hip_conv_f32", C.byref(d), util.ptr(dX), util.ptr(dW), util.ptr(db), R.ACT_RELU, C.c_float(0), util.ptr(dY), None, util.ptr(dX))
    rt.sync()
    lin = ob.conv_f32(X, Wt, b, pads=(1, 1, 1, 1), strides=(1, 1), dils=(1, 1), group=1, act=0)
    want = ob.unary(ob.add_broadcast(lin, X), R.ACT_RELU, 0.0)
    got = util.to_host(dY)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5) and (got > 0).any() and (got == 0).any()


def test_hard_sigmoid_hard_swish_and_swish(rt):
    x = np.concatenate([util.normal(452, 1000 + 3, 2.5), np.array([-3.0, 3.0, -2.5, 2.5, 0.0, -0.0], np.float32)])
    for ops, exact in [([(R.ACT_HARDSIGMOID, 0.2, 0.5)], True), ([(R.ACT_HARDSIGMOID, 0.37, 0.1)], True), ([(R.ACT_HARDSWISH, 0.0, 0.0)], True),
                       ([(R.ACT_SWISH, 0.0, 0.0)], False), ([(R.ACT_SWISH, 0.0, 0.0), (R.ACT_HARDSWISH, 0.0, 0.0), (R.ACT_HARDSIGMOID, 0.2, 0.5)], False)]:
        got, want = run_chain(rt, x, ops), ob.unary_chain(x, ops)
        if exact:       # multiplications, additions and clamps only: the device computes the reference's bits
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), ops
        else:
            assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(1.0, np.abs(want))), ops
    x64 = x.astype(np.float64)
    assert np.allclose(run_chain(rt, x, [(R.ACT_SWISH, 0.0, 0.0)]), x64 / (1 + np.exp(-x64)), rtol=1e-5, atol=1e-6)
    # the single-operator entry point takes the codes too (HardSigmoid's beta only through the chain)
    dx, dy = util.to_dev(x), util.dev_empty(x.shape, np.float32)
    rt.call("sofie_hip_unary_f32", util.ptr(dy), util.ptr(dx), C.c_size_t(x.size), R.ACT_HARDSWISH, C.c_float(0))
    rt.sync()
    assert np.array_equal(util.to_host(dy).view(np.uint32), ob.unary(x, R.ACT_HARDSWISH, 0.0).view(np.uint32))


def test_selu(rt):
    x = util.normal(450, 1000 + 3, 2.0)
    alpha, gamma = 1.6732631921768188, 1.0507010221481323
    got = run_chain(rt, x, [(R.ACT_SELU, alpha, gamma)])
    want = ob.unary_chain(x, [(R.ACT_SELU, alpha, gamma)])
    ref = gamma * (np.maximum(0, x.astype(np.float64)) + np.minimum(0, alpha * (np.exp(x.astype(np.float64)) - 1)))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6) and np.allclose(want, ref, rtol=1e-5, atol=1e-6)


def test_elu_and_erf(rt):
    x = util.normal(451, 1000 + 3, 2.0)
    got = run_chain(rt, x, [(R.ACT_ELU, 0.7, 0.0)])
    want = ob.unary_chain(x, [(R.ACT_ELU, 0.7, 0.0)])
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6) and np.array_equal(got[x >= 0], x[x >= 0]) and (got < 0).any()
    got = run_chain(rt, x, [(R.ACT_ERF, 0.0, 0.0), (R.ACT_ELU, 1.0, 0.0)])
    want = ob.unary_chain(x, [(R.ACT_ERF, 0.0, 0.0), (R.ACT_ELU, 1.0, 0.0)])
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6) and want.std() > 0.1

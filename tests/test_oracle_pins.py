"""Pins for the parts of the oracle the golden fixtures do not reach: closed forms, brute force in
float64 / int64, exhaustive tables, the reference's literal test values, and the reference's own
memory planner (oracle/_ref) where it is built."""
import ctypes as C
import itertools

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import util


# ---- fp32 Gemm: literals of the reference's constant-folding / MatMul tests --------------------------------

def test_gemm_literals_of_the_reference_tests():
    # Gemm_ConstantFolding: A=[[1,2,3],[4,5,6]] x B=[[7,8],[9,10],[11,12]] + C=[[1,1],[1,1]] -> {59,65,140,155}
    # (tests/cpu/TestCustomModelsFromONNX.cxx:509-527)
    A = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    B = np.arange(7, 13, dtype=np.float32).reshape(3, 2)
    Cb = np.ones((2, 2), dtype=np.float32)
    y = ob.gemm_f32(A, B, Cb, M=2, N=2, K=3, bias_mode=4)
    assert y.ravel().tolist() == [59, 65, 140, 155]
    # ExternalStream model: Gemm+Relu of ones[1,3]... = 3.5 (tests/alpaka/TestAlpakaExternalStream.cxx:34-37):
    # x = ones(3), W = 1, b = 0.5
    y = ob.gemm_f32(np.ones((1, 3), np.float32), np.ones((3, 1), np.float32), np.array([0.5], np.float32), M=1, N=1, K=3,
                    bias_mode=1, act=1)
    assert y[0, 0] == 3.5


@pytest.mark.parametrize("transA,transB,bias_mode,act", list(itertools.product([0, 1], [0, 1], [0, 1, 2, 3, 4], [0, 1, 2])))
def test_gemm_f32_against_float64_brute_force(transA, transB, bias_mode, act):
    M, N, K = 7, 5, 11
    A = util.normal(1, M * K).reshape((K, M) if transA else (M, K))
    B = util.normal(2, N * K).reshape((N, K) if transB else (K, N))
    Cshape = {0: None, 1: (N,), 2: (M, 1), 3: (1,), 4: (M, N)}[bias_mode]
    Cb = None if Cshape is None else util.normal(3, int(np.prod(Cshape))).reshape(Cshape)
    alpha, beta = 0.75, 2.0
    got = ob.gemm_f32(A, B, Cb, M=M, N=N, K=K, transA=transA, transB=transB, alpha=alpha, beta=beta, bias_mode=bias_mode,
                      act=act, act_alpha=0.3)
    opA = (A.T if transA else A).astype(np.float64)
    opB = (B.T if transB else B).astype(np.float64)
    ref = alpha * (opA @ opB)
    if bias_mode in (1, 2, 3):
        ref = ref + Cb.astype(np.float64)  # broadcast bias: beta is forced to 1 (ROperator_Gemm.hxx:580)
    elif bias_mode == 4:
        ref = ref + beta * Cb.astype(np.float64)
    if act == 1:
        ref = np.maximum(ref, 0)
    elif act == 2:
        ref = np.where(ref >= 0, ref, 0.3 * ref)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)


def test_relu_special_values():
    x = np.array([np.nan, -0.0, 0.0, -1.0, 2.5, np.inf, -np.inf], dtype=np.float32)
    y = ob.unary(x, 1)
    assert y.tolist() == [0.0, 0.0, 0.0, 0.0, 2.5, np.inf, 0.0]
    assert not np.signbit(y[1])  # -0 -> +0 as on the reference's CPU path


def test_activations_closed_forms():
    import math
    x = np.linspace(-4, 4, 33, dtype=np.float32)
    assert np.allclose(ob.unary(x, 3), 1 / (1 + np.exp(-x.astype(np.float64))), atol=1e-6)
    assert np.allclose(ob.unary(x, 4), [0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in x.astype(np.float64)], atol=1e-6)
    assert np.allclose(ob.unary(x, 5), [0.5 * v * (1 + math.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3))) for v in x.astype(np.float64)], atol=1e-6)
    assert np.allclose(ob.unary(x, 2, 0.1), np.where(x >= 0, x, 0.1 * x))
    assert np.allclose(ob.unary(x, 6), np.tanh(x.astype(np.float64)), atol=1e-6)


# ---- im2col / conv: direct 7-loop convolution in float64 -----------------------------------------------------

def direct_conv(X, W, b, pads, strides, dils, group):
    N, Cc, H, Wd = X.shape
    Cout, Cg, kh, kw = W.shape
    OH, OW = ob.conv_out_hw(H, Wd, kh, kw, pads, strides, dils)
    Y = np.zeros((N, Cout, OH, OW))
    for n, co, oh, ow in itertools.product(range(N), range(Cout), range(OH), range(OW)):
        g = co // (Cout // group)
        s = 0.0 if b is None else float(b[co])
        for ci, y, x in itertools.product(range(Cg), range(kh), range(kw)):
            ih, iw = oh * strides[0] - pads[0] + y * dils[0], ow * strides[1] - pads[1] + x * dils[1]
            if 0 <= ih < H and 0 <= iw < Wd:
                s += float(X[n, g * Cg + ci, ih, iw]) * float(W[co, ci, y, x])
        Y[n, co, oh, ow] = s
    return Y


@pytest.mark.parametrize("case", [
    (1, 1, 5, 5, 1, 3, 3, (1, 1, 1, 1), (1, 1), (1, 1), 1), (2, 4, 6, 7, 6, 3, 2, (1, 0, 2, 1), (2, 1), (1, 1), 2),
    (1, 2, 9, 9, 4, 3, 3, (2, 2, 2, 2), (1, 1), (2, 2), 1), (2, 3, 1, 12, 4, 1, 5, (0, 2, 0, 2), (1, 2), (1, 1), 1),
    (1, 6, 5, 5, 6, 3, 3, (1, 1, 1, 1), (1, 1), (1, 2), 3)])
def test_conv_f32_equals_direct_convolution(case):
    N, Cc, H, W, Cout, kh, kw, pads, strides, dils, group = case
    X = util.normal(5, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.normal(6, Cout * (Cc // group) * kh * kw).reshape(Cout, Cc // group, kh, kw)
    b = util.normal(7, Cout)
    for bias in (None, b):
        got = ob.conv_f32(X, Wt, bias, pads=pads, strides=strides, dils=dils, group=group)
        assert np.allclose(got, direct_conv(X, Wt, bias, pads, strides, dils, group), rtol=1e-5, atol=1e-5)


def direct_conv3d(X, W, b, pads, strides, dils, group):
    N, Cc = X.shape[:2]
    Cout, Cg = W.shape[:2]
    sp, k = X.shape[2:], W.shape[2:]
    out = [(sp[a] + pads[a] + pads[a + 3] - (dils[a] * (k[a] - 1) + 1)) // strides[a] + 1 for a in range(3)]
    Y = np.zeros((N, Cout, *out))
    for n, co, od, oh, ow in itertools.product(range(N), range(Cout), *[range(o) for o in out]):
        g = co // (Cout // group)
        s = 0.0 if b is None else float(b[co])
        for ci, z, y, x in itertools.product(range(Cg), *[range(v) for v in k]):
            pos = [o * strides[a] - pads[a] + t * dils[a] for a, (o, t) in enumerate(zip((od, oh, ow), (z, y, x)))]
            if all(0 <= pos[a] < sp[a] for a in range(3)):
                s += float(X[n, g * Cg + ci, pos[0], pos[1], pos[2]]) * float(W[co, ci, z, y, x])
        Y[n, co, od, oh, ow] = s
    return Y


CONV3D_CASES = [
    # N, C, (D,H,W), Cout, (kd,kh,kw), pads {d0,h0,w0,d1,h1,w1}, strides, dils, group
    (1, 1, (3, 4, 4), 2, (2, 3, 3), (0, 1, 1, 0, 1, 1), (1, 1, 1), (1, 1, 1), 1),
    (2, 4, (5, 6, 7), 6, (3, 2, 3), (1, 0, 2, 0, 1, 1), (2, 1, 2), (1, 1, 1), 2),
    (1, 2, (7, 5, 6), 3, (2, 3, 2), (2, 1, 0, 1, 2, 1), (1, 2, 1), (2, 1, 2), 1),
    (1, 6, (4, 4, 4), 6, (3, 3, 3), (1, 1, 1, 1, 1, 1), (1, 1, 1), (1, 1, 1), 3),
]


@pytest.mark.parametrize("case", CONV3D_CASES)
def test_conv3d_f32_equals_direct_convolution(case):
    # every axis has its own extent, kernel, pad pair, stride and dilation somewhere in the cases, so an axis mix-up shows
    N, Cc, sp, Cout, k, pads, strides, dils, group = case
    X = util.normal(15, N * Cc * int(np.prod(sp))).reshape(N, Cc, *sp)
    Wt = util.normal(16, Cout * (Cc // group) * int(np.prod(k))).reshape(Cout, Cc // group, *k)
    b = util.normal(17, Cout)
    for bias in (None, b):
        got = ob.conv3d_f32(X, Wt, bias, pads=pads, strides=strides, dils=dils, group=group)
        want = direct_conv3d(X, Wt, bias, pads, strides, dils, group)
        assert got.shape == want.shape
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


def test_conv3d_of_depth_one_is_the_2d_convolution():
    X = util.normal(18, 2 * 3 * 6 * 5).reshape(2, 3, 1, 6, 5)
    Wt = util.normal(19, 4 * 3 * 3 * 2).reshape(4, 3, 1, 3, 2)
    got = ob.conv3d_f32(X, Wt, None, pads=(0, 1, 0, 0, 2, 1), strides=(1, 2, 1), dils=(1, 1, 2), group=1)
    want = ob.conv_f32(X[:, :, 0], Wt[:, :, 0], None, pads=(1, 0, 2, 1), strides=(2, 1), dils=(1, 2), group=1)
    assert np.array_equal(got[:, :, 0], want)


def test_im2col_layout():
    # rows (c,kh,kw), columns (oh,ow), zero outside the image
    x = np.arange(2 * 3 * 3, dtype=np.float32).reshape(2, 3, 3)
    col = ob.im2col(x, 2, 2, (1, 0, 0, 0), (1, 1), (1, 1))  # pad one row on top
    assert col.shape == (8, 6)
    assert col[0].tolist() == [0, 0, 3 * 0 + 0, 1, 3, 4]      # c=0,kh=0,kw=0: first output row reads the padding
    assert col[3].tolist() == [1, 2, 4, 5, 7, 8]              # c=0,kh=1,kw=1
    assert col[4].tolist() == [0, 0, 9, 10, 12, 13]           # c=1,kh=0,kw=0


# ---- the CPU path's greedy pool planner ------------------------------------------------------------------------

def check_greedy_plan(ops, sizes, plan, model_outputs=()):
    """Tensors alive at the same time do not share bytes, and everything lies inside the pool.  A tensor is alive from its
    producer until after its last reader (until the end for a model output)."""
    prod = {t: i for i, (outs, ins) in enumerate(ops) for t in outs}
    last = plan["last_use"]
    end = lambda t: len(ops) if last[t] < 0 else last[t]
    off = plan["offsets"]
    for a in prod:
        assert off[a] + sizes[a] <= plan["pool_bytes"]
        for b in prod:
            if a < b and prod[a] <= end(b) and prod[b] <= end(a):  # alive together at some operator (released AFTER the last reader ran)
                assert off[a] + sizes[a] <= off[b] or off[b] + sizes[b] <= off[a], (a, b)


def test_greedy_planner_linear16_is_two_buffers_of_3200():
    # the reference's CPU Session of Linear_16: 10 Gemm(+Relu) operators, outputs 9 x [16,50] and [16,10], fp32;
    # its generated pool is std::vector<char>(6400): two 3200-byte buffers used in turn
    sizes = [3200] * 9 + [640]
    ops = [([i], [i - 1]) for i in range(10)]  # operator 0 reads the model input (id -1)
    plan = ob.plan_memory_greedy(ops, sizes, model_outputs=[9])
    assert plan["pool_bytes"] == 6400
    assert plan["offsets"][:9] == [0, 3200] * 4 + [0]
    assert plan["offsets"][9] == 3200 + 3200 - 640   # cut from the END of the free chunk
    check_greedy_plan(ops, sizes, plan, [9])


def test_greedy_planner_hand_worked_cases():
    # outputs of one operator are placed largest first; a tensor nothing reads is released by its own producer
    ops = [([0, 1], [-1]), ([2], [1]), ([3], [2, 0])]
    sizes = [100, 300, 50, 400]
    plan = ob.plan_memory_greedy(ops, sizes, model_outputs=[3])
    # op 0: tensor 1 (300) at 0, tensor 0 (100) at 300.  op 1: tensor 2 (50) appended at 400, then tensor 1 is released: free [0,300).
    # op 2: tensor 3 (400) does not fit [0,300), which is not the last chunk either: appended at 450; pool 850.
    assert plan["offsets"] == [300, 0, 400, 450] and plan["pool_bytes"] == 850
    # a free last chunk grows: A(100) released, then B(500) takes its place and the pool is 500, not 600
    ops = [([0], [-1]), ([1], [0]), ([2], [1])]
    plan = ob.plan_memory_greedy(ops, [100, 64, 500], model_outputs=[2])
    # op 1: tensor 1 appended at 100, tensor 0 released: free [0,100).  op 2: 500 > 100 and the free chunk is not the last one:
    # appended at 164; then tensor 1 released and merged with [0,100): free [0,164)
    assert plan["offsets"] == [0, 100, 164] and plan["pool_bytes"] == 664
    ops = [([0], [-1]), ([1], [-1]), ([2], [0, 1]), ([3], [2])]
    plan = ob.plan_memory_greedy(ops, [100, 200, 40, 900], model_outputs=[3])
    # op 2: tensor 2 at 300; tensors 0 and 1 released and merged: free [0,300).  op 3: 900 > 300; the free chunk [0,300) is the last
    # free one but not the last of the pool ([300,340) is tensor 2): appended at 340; pool 1240
    assert plan["offsets"] == [0, 100, 300, 340] and plan["pool_bytes"] == 1240
    ops = [([0], [-1]), ([1], [0]), ([2], [-1])]
    plan = ob.plan_memory_greedy(ops, [100, 50, 700], model_outputs=[2])
    # a tensor nobody reads is never given back (only an operator's INPUTS are released): tensor 1 stays at [100,150), the free
    # chunk [0,100) is not the last of the pool, tensor 2 is appended at 150
    assert plan["offsets"] == [0, 100, 150] and plan["pool_bytes"] == 850
    ops = [([0], [-1]), ([1], [0]), ([2], [1]), ([3], [2])]
    plan = ob.plan_memory_greedy(ops, [100, 50, 30, 500], model_outputs=[3])
    # op 1: tensor 1 at 100, tensor 0 released: free [0,100).  op 2: tensor 2 (30) is cut from the END of that chunk: [70,100); tensor 1
    # released: free [0,70) and [100,150).  op 3: 500 fits neither, but [100,150) is the last free chunk AND the last of the pool:
    # it grows in place; pool 600
    assert plan["offsets"] == [0, 100, 70, 100] and plan["pool_bytes"] == 600


@pytest.mark.parametrize("seed", range(30))
def test_greedy_planner_never_overlaps_live_tensors(seed):
    rng = np.random.default_rng(seed)
    n_ops = int(rng.integers(3, 25))
    ops, sizes, made = [], [], []
    for i in range(n_ops):
        k = int(rng.integers(1, 4))
        outs = list(range(len(sizes), len(sizes) + k))
        sizes += [int(rng.integers(1, 40)) * 16 for _ in range(k)]
        ins = [int(t) for t in rng.choice(made, size=min(len(made), int(rng.integers(0, 4))), replace=False)] if made else [-1]
        ops.append((outs, ins or [-1]))
        made += outs
    outputs = [made[-1]]
    plan = ob.plan_memory_greedy(ops, sizes, model_outputs=outputs)
    check_greedy_plan(ops, sizes, plan, outputs)
    # never smaller than what is alive at once, never larger than everything laid end to end
    prod = {t: i for i, (outs, ins) in enumerate(ops) for t in outs}
    last = plan["last_use"]
    peak = max(sum(sizes[t] for t in prod if prod[t] <= i and (last[t] < 0 or last[t] >= i)) for i in range(n_ops))
    assert peak <= plan["pool_bytes"] <= sum(sizes)


# ---- memory planner -----------------------------------------------------------------------------------------

def check_plan(begin, end, size, plan):
    off, total = plan["offsets"], plan["total_bytes"]
    for i in range(len(begin)):
        assert off[i] + size[i] <= total
        for j in range(i):
            if begin[i] < end[j] and begin[j] < end[i]:  # live together
                assert off[i] + size[i] <= off[j] or off[j] + size[j] <= off[i], (i, j)


def linear16_lifetimes(row_bytes):
    # 10 chained Gemm(+Relu) operators, outputs [16,50] x9 then [16,10]; output i is produced by op i and last
    # read by op i+1 -> lifetime [i, i+2).  The reference plans these into 2 x 3328 = 6656 bytes (256-byte aligned).
    n = 10
    begin = list(range(n))
    end = [i + 2 for i in range(n)]
    size = [row_bytes] * 9 + [768]
    return begin, end, size


def test_planner_linear16_known_total():
    begin, end, size = linear16_lifetimes(3328)  # 16*50*4 = 3200 rounded up to 256
    plan = ob.organize_memory(begin, end, size)
    check_plan(begin, end, size, plan)
    assert plan["total_bytes"] == 6656


def test_planner_rejects_empty_lifetime():
    with pytest.raises(ValueError):
        ob.organize_memory([0, 3], [1, 3], [16, 16])


def test_planner_equals_reference_planner():
    ref = ob.load_ref_planner()
    if ref is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    rng = np.random.default_rng(7)
    cases = [linear16_lifetimes(3328)]
    for _ in range(200):
        n = int(rng.integers(1, 9))  # <= 16 events: std::sort is an insertion sort there, i.e. equal events keep tensor order
        begin = [int(v) for v in rng.integers(0, 12, n)]
        end = [b + int(v) for b, v in zip(begin, rng.integers(1, 6, n))]
        size = [int(v) * 256 for v in rng.integers(1, 9, n)]
        cases.append((begin, end, size))
    for begin, end, size in cases:
        mine = ob.organize_memory(begin, end, size)
        theirs = ob.organize_memory(begin, end, size, lib=ref, fn="ref_organize_memory")
        check_plan(begin, end, size, mine)
        check_plan(begin, end, size, theirs)
        if len(begin) <= 8:
            assert mine == theirs
    # larger plans: the reference leaves the order of equal events to std::sort, so only the invariants
    # (no overlap of live tensors, everything inside the pool) are compared
    for _ in range(50):
        n = int(rng.integers(9, 40))
        begin = [int(v) for v in rng.integers(0, 30, n)]
        end = [b + int(v) for b, v in zip(begin, rng.integers(1, 8, n))]
        size = [int(v) * 256 for v in rng.integers(1, 9, n)]
        mine = ob.organize_memory(begin, end, size)
        theirs = ob.organize_memory(begin, end, size, lib=ref, fn="ref_organize_memory")
        check_plan(begin, end, size, mine)
        check_plan(begin, end, size, theirs)
        lower = max(sum(sz for b, e, sz in zip(begin, end, size) if b <= t < e) for t in range(40))
        assert mine["total_bytes"] >= lower and theirs["total_bytes"] >= lower


# ---- quantised operators (ONNX definitions) ------------------------------------------------------------------

def test_quantize_linear_ties_saturation_nan():
    s = np.float32(0.5)
    x = np.array([0.25, 0.75, 1.25, -0.25, -0.75, 63.75, 100.0, -64.25, -100.0, np.nan, np.inf, -np.inf, 0.0], dtype=np.float32)
    q = ob.quantize_linear(x, s)
    #            0.5->0  1.5->2  2.5->2  -0.5->0  -1.5->-2  127.5->128->127  sat  -128.5->-128  sat  nan->0  +-inf sat
    assert q.tolist() == [0, 2, 2, 0, -2, 127, 127, -128, -128, 0, 127, -128, 0]
    xs = util.normal(3, 10000, 3.0)
    sc = np.float32(0.0371)
    want = np.clip(np.rint(xs / sc), -128, 127).astype(np.int8)  # numpy: fp32 divide, round half to even
    assert np.array_equal(ob.quantize_linear(xs, sc), want)
    assert np.array_equal(ob.dequantize_linear(want, sc), want.astype(np.float32) * sc)


def test_all_int8_products_and_matmul_integer():
    a = np.arange(-128, 128, dtype=np.int8)
    A = np.repeat(a, 256).reshape(-1, 1)      # [65536,1]
    B = np.tile(a, 256).reshape(-1, 1)        # B^T rows
    # K = 1: acc[m, n] with m == n enumerates all 65536 products
    acc = ob.matmul_integer(A[:512], B[:512], M=512, N=512, K=1, transB=1)
    assert np.array_equal(acc, A[:512].astype(np.int32) @ B[:512].astype(np.int32).T)
    prod = np.array([ob.matmul_integer(A[i:i + 1], B[i:i + 1], M=1, N=1, K=1, transB=1)[0, 0] for i in range(0, 65536, 257)])
    assert np.array_equal(prod, (A[::257, 0].astype(np.int32) * B[::257, 0].astype(np.int32)))
    for (M, N, K, tA, tB) in [(5, 7, 3, 0, 0), (9, 4, 33, 1, 0), (6, 6, 64, 0, 1), (3, 8, 17, 1, 1)]:
        X = util.int8_sym(1, M * K).reshape((K, M) if tA else (M, K))
        Y = util.int8_sym(2, N * K).reshape((N, K) if tB else (K, N))
        ref = (X.T if tA else X).astype(np.int64) @ (Y.T if tB else Y).astype(np.int64)
        assert np.array_equal(ob.matmul_integer(X, Y, M=M, N=N, K=K, transA=tA, transB=tB), ref)
        assert np.array_equal(ob.matmul_integer(X, Y, M=M, N=N, K=K, transA=tA, transB=tB, omp=True), ref)
    # identity and one-hot special cases
    I = np.eye(16, dtype=np.int8)
    X = util.int8_sym(3, 16 * 16).reshape(16, 16)
    assert np.array_equal(ob.matmul_integer(X, I, M=16, N=16, K=16), X.astype(np.int32))


def test_requant_epilogue_definition():
    acc = np.array([[1, 3, 5, -1, -3, 255, -257, 1000, -1000, 0]], dtype=np.int32)
    got = ob.gemm_i8_epilogue(acc, scale_scalar=np.float32(0.5), out=2)
    assert got.tolist() == [[0, 2, 2, 0, -2, 127, -128, 127, -128, 0]]  # ties to even, saturation
    got = ob.gemm_i8_epilogue(acc, scale_scalar=np.float32(0.5), out=2, relu_out=1)
    assert got.tolist() == [[0, 2, 2, 0, 0, 127, 0, 127, 0, 0]]
    bias = np.arange(10, dtype=np.int32)
    got = ob.gemm_i8_epilogue(acc, bias=bias, out=0, relu_acc=1)
    assert got.tolist() == [np.maximum(acc[0] + bias, 0).tolist()]  # bias added in int32 before anything else
    # int32 -> fp32 is round-to-nearest-even above 2^24
    big = np.array([[(1 << 24) + 1, (1 << 24) + 3, -(1 << 24) - 1]], dtype=np.int32)
    got = ob.gemm_i8_epilogue(big, scale_scalar=np.float32(1.0), out=1)
    assert got.tolist() == [[float(1 << 24), float((1 << 24) + 4), -float(1 << 24)]]
    # DequantizeLinear followed by QuantizeLinear == the two separate operators
    acc = util.int32_range(5, 4096, -200000, 200000).reshape(64, 64)
    s, qs = np.float32(3.1e-4), np.float32(0.27)
    fused = ob.gemm_i8_epilogue(acc, scale_scalar=s, q_scale=qs, out=3, relu_acc=1)
    two = ob.quantize_linear(ob.dequantize_linear(np.maximum(acc, 0), s), qs)
    assert np.array_equal(fused, two)


def test_conv_i8_equals_float_conv_of_integers():
    N, Cc, H, W, Cout, kh, kw = 2, 4, 6, 5, 6, 3, 3
    X = util.int8_sym(8, N * Cc * H * W).reshape(N, Cc, H, W)
    Wt = util.int8_sym(9, Cout * 2 * kh * kw).reshape(Cout, 2, kh, kw)
    bias = util.int32_range(10, Cout, -500, 500)
    got = ob.conv_i8(X, Wt, bias, None, pads=(1, 1, 1, 1), strides=(1, 2), dils=(1, 1), group=2, out=0)
    ref = direct_conv(X.astype(np.float64), Wt.astype(np.float64), bias.astype(np.float64), (1, 1, 1, 1), (1, 2), (1, 1), 2)
    assert np.array_equal(got, ref.astype(np.int32))


def test_e4m3_codec_exhaustive():
    codes = np.arange(256, dtype=np.uint8)
    vals = ob.e4m3_to_f32(codes)
    # OCP e4m3fn: 0x7f/0xff NaN, max 448, smallest subnormal 2^-9, no infinities
    assert np.isnan(vals[0x7F]) and np.isnan(vals[0xFF]) and np.isfinite(np.delete(vals, [0x7F, 0xFF])).all()
    assert vals[0x7E] == 448 and vals[0x01] == 2.0 ** -9 and vals[0x08] == 2.0 ** -6 and vals[0x38] == 1.0 and vals[0xB8] == -1.0
    for c in range(256):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        if e == 15 and m == 7:
            continue
        want = (m / 8 * 2.0 ** -6) if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        assert vals[c] == (-want if s else want)
    finite = np.isfinite(vals)
    assert np.array_equal(ob.quantize_fp8(vals[finite], 1.0), codes[finite])  # every value encodes to itself
    pos = np.sort(vals[finite & ~np.signbit(vals)])
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    enc = ob.quantize_fp8(mids, 1.0)
    assert (enc & 1 == 0).all()  # a midpoint goes to the neighbour with the even mantissa
    lo, hi = ob.quantize_fp8(np.nextafter(mids, np.float32(0)), 1.0), ob.quantize_fp8(np.nextafter(mids, np.float32(1e9)), 1.0)
    assert np.array_equal(ob.e4m3_to_f32(lo), pos[:-1]) and np.array_equal(ob.e4m3_to_f32(hi), pos[1:])
    assert ob.quantize_fp8(np.array([448, 464, 465, 1e30, np.inf, -np.inf, np.nan], np.float32), 1.0).tolist() == [0x7E, 0x7E, 0x7E, 0x7E, 0x7E, 0xFE, 0x7F]


def test_bf16_rounding():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.0, 3.4e38, np.inf], dtype=np.float32)
    #             exact  tie->even(1.0)  tie->even(1.015625)
    got = ob.bf16_bits_to_f32(ob.f32_to_bf16_bits(x))
    assert got.tolist() == [1.0, 1.0, 1.015625, -3.0, np.inf, np.inf]


def test_gemm_fp8_arbiter_is_exact_on_small_integers():
    # small integers are exact in e4m3 and their dot products are exact in float
    A = (util.int8_sym(11, 8 * 32).reshape(8, 32) % 5).astype(np.float32)
    B = (util.int8_sym(12, 6 * 32).reshape(6, 32) % 4).astype(np.float32)
    got = ob.gemm_fp8(ob.quantize_fp8(A, 1.0), ob.quantize_fp8(B, 1.0), M=8, N=6, K=32, transB=1, scale=1.0, out=1)
    assert np.array_equal(got, A @ B.T)


def test_global_avg_pool_i8():
    X = util.int8_sym(13, 2 * 3 * 20).reshape(2, 3, 20)
    got = ob.global_avg_pool_i8(X, np.float32(0.05))
    want = (X.astype(np.int64).sum(-1).astype(np.float32) * np.float32(0.05)) / np.float32(20)
    assert np.array_equal(got, want)


def test_batchnorm_closed_forms():
    # x == mean gives the bias; gamma == sqrt(var + eps) gives x - mean + bias; float64 arbiter for the general case
    Cc = 5
    mean, beta = util.normal(301, Cc), util.normal(302, Cc)
    var = (0.2 + util.uniform01(303, Cc)).astype(np.float32)
    X = np.broadcast_to(mean[None, :, None], (3, Cc, 4)).copy()
    y, _ = ob.batchnorm(X, np.ones(Cc, np.float32), beta, mean, var)
    assert np.array_equal(y, np.broadcast_to(beta[None, :, None], y.shape))
    X = util.normal(304, 3 * Cc * 4).reshape(3, Cc, 4)
    gamma = util.normal(305, Cc)
    y, fused = ob.batchnorm(X, gamma, beta, mean, var, eps=1e-3)
    ref = (X.astype(np.float64) - mean[None, :, None]) * (gamma.astype(np.float64) / np.sqrt(var.astype(np.float64) + 1e-3))[None, :, None] + beta[None, :, None]
    assert np.abs(y - ref).max() <= 1e-6 * (1 + np.abs(ref).max())
    assert np.allclose(fused, gamma / np.sqrt(var + np.float32(1e-3)), rtol=1e-6)
    yr, _ = ob.batchnorm(X, gamma, beta, mean, var, eps=1e-3, relu=1)
    assert np.array_equal(yr, np.where(y > 0, y, np.float32(0)))


# ---- the other one-to-one operators: pinned by numpy's routines and by identities ----------------------------

def test_basic_unary_operators_against_library_routines_and_identities():
    """Codes 7..21 (ROperator_BasicUnary.hxx:17-103, ROperator_Clip.hxx:18).  numpy's float32 routines are an independent
    implementation; the identities catch a swapped code (exp for log, sin for cos, asinh for acosh ...)."""
    from tests import util
    z = util.normal(501, 4000, 2.0)
    u = util.uniform01(502, 4000)
    pos = (0.01 + 50 * u).astype(np.float32)
    lib = {7: (np.where(z >= 0, 0.1 + np.abs(z), -0.1 - np.abs(z)).astype(np.float32), lambda x: np.float32(1) / x), 8: (9 * u, np.sqrt),
           9: (z, np.negative), 10: (z, np.exp), 11: (pos, np.log), 12: (z, np.sin), 13: (z, np.cos), 14: (z, np.abs),
           15: (12 * z, lambda x: np.where(x >= 20, x, np.log1p(np.exp(x.astype(np.float64))))), 16: (z, np.arctan), 17: (3 * z, np.floor),
           18: (z, np.arcsinh), 19: ((1 + 20 * u).astype(np.float32), np.arccosh), 20: (((u - 0.5) * 1.9).astype(np.float32), np.arctanh)}
    for code, (x, f) in lib.items():
        x = x.astype(np.float32)
        got = ob.unary(x, code, 0.0)
        want = f(x.astype(np.float64) if code not in (7,) else x).astype(np.float64)
        assert np.all(np.abs(got - want) <= 2e-6 * np.maximum(1.0, np.abs(want))), code
    # identities
    assert np.allclose(ob.unary(ob.unary(pos, 11, 0), 10, 0), pos, rtol=2e-5)                     # exp(log x) = x
    s, c = ob.unary(z, 12, 0).astype(np.float64), ob.unary(z, 13, 0).astype(np.float64)
    assert np.allclose(s * s + c * c, 1.0, atol=1e-6)                                               # sin^2 + cos^2 = 1
    assert np.allclose(np.sinh(ob.unary(z, 18, 0).astype(np.float64)), z, rtol=1e-5, atol=1e-6)     # sinh(asinh x) = x
    big = (1 + 20 * u).astype(np.float32)
    assert np.allclose(np.cosh(ob.unary(big, 19, 0).astype(np.float64)), big, rtol=1e-5)            # cosh(acosh x) = x
    assert np.allclose(np.tan(ob.unary(z, 16, 0).astype(np.float64)), z, rtol=1e-5, atol=1e-6)      # tan(atan x) = x
    assert np.array_equal(ob.unary(np.array([25.0, 20.0], np.float32), 15, 0), np.array([25.0, 20.0], np.float32))  # softplus: identity from 20 on
    assert abs(float(ob.unary(np.array([0.0], np.float32), 15, 0)[0]) - np.log(2.0)) < 1e-7
    # Clip: the lower bound wins when the bounds cross (max(lo, min(hi, x))), bounds are attained exactly
    x = np.array([-2, -0.25, 0, 0.75, 3], np.float32)
    assert np.array_equal(ob.unary_chain(x, [(21, -0.25, 0.75)]), np.array([-0.25, -0.25, 0, 0.75, 0.75], np.float32))
    assert np.array_equal(ob.unary_chain(x, [(21, 1.0, 0.5)]), np.full(5, 1.0, np.float32))


def test_unary_chain_is_applied_left_to_right():
    from tests import util
    x = util.normal(503, 100, 1.0)
    ops = [(2, 0.1, 0.0), (10, 0.0, 0.0), (21, 0.5, 3.0), (11, 0.0, 0.0)]          # LeakyRelu, Exp, Clip, Log
    want = x.copy()
    for o in ops:
        want = ob.unary_chain(want, [o])
    assert np.array_equal(ob.unary_chain(x, ops), want)
    ref = np.log(np.clip(np.exp(np.where(x >= 0, x, np.float32(0.1) * x).astype(np.float64)), 0.5, 3.0))
    assert np.allclose(want, ref, rtol=1e-5, atol=1e-6)
    # not commutative: the reverse order gives something else
    assert not np.allclose(ob.unary_chain(x, ops[::-1]), want, equal_nan=True)
    assert np.array_equal(ob.unary_chain(x, []), x)


def _pool_by_definition(X, mode, k, pads, strides, ceil_mode, include_pad):
    """ONNX MaxPool / AveragePool written from the specification: pad the image (-inf for max; zeros plus a validity
    mask for the average), slice each window, reduce in float64."""
    N, Cc, H, W = X.shape
    (kh, kw), (ph0, pw0, ph1, pw1), (sh, sw) = k, pads, strides

    def extent(n, p0, p1, kk, s):
        span = n + p0 + p1 - kk
        out = -(-span // s) + 1 if ceil_mode else span // s + 1
        if ceil_mode and (out - 1) * s >= n + p0:   # a window may not start in the end padding
            out -= 1
        return out
    OH, OW = extent(H, ph0, ph1, kh, sh), extent(W, pw0, pw1, kw, sw)
    big_h, big_w = (OH - 1) * sh + kh, (OW - 1) * sw + kw     # the padded canvas every window fits into
    canvas = np.full((N, Cc, max(big_h, H + ph0), max(big_w, W + pw0)), -np.inf if mode == "max" else 0.0)
    real = np.zeros(canvas.shape[2:], dtype=bool)     # true input samples
    padded = np.zeros(canvas.shape[2:], dtype=bool)   # input plus the declared padding
    canvas[:, :, ph0:ph0 + H, pw0:pw0 + W] = X
    real[ph0:ph0 + H, pw0:pw0 + W] = True
    padded[:H + ph0 + ph1, :W + pw0 + pw1] = True
    Y = np.empty((N, Cc, OH, OW))
    for oh, ow in itertools.product(range(OH), range(OW)):
        win = canvas[:, :, oh * sh:oh * sh + kh, ow * sw:ow * sw + kw]
        if mode == "max":
            Y[:, :, oh, ow] = win.max(axis=(2, 3))
        else:
            count = (padded if include_pad else real)[oh * sh:oh * sh + kh, ow * sw:ow * sw + kw].sum()
            Y[:, :, oh, ow] = win.sum(axis=(2, 3)) / count
    return Y


@pytest.mark.parametrize("mode", ["max", "average"])
def test_pool_equals_the_definition_on_a_sweep_of_geometries(mode):
    rng = np.random.default_rng(11)
    seen_ceil_overhang = 0
    for case in range(120):
        H, W = rng.integers(3, 12, 2)
        kh, kw = rng.integers(1, 5, 2)
        sh, sw = rng.integers(1, 4, 2)
        pads = tuple(int(min(p, kk - 1)) for p, kk in zip(rng.integers(0, 3, 4), (kh, kw, kh, kw)))  # ONNX: pad < kernel
        ceil_mode, include_pad = int(case % 2), int((case // 2) % 2)
        X = rng.standard_normal((2, 3, H, W)).astype(np.float32)
        want = _pool_by_definition(X.astype(np.float64), mode, (kh, kw), pads, (sh, sw), ceil_mode, include_pad)
        got = ob.pool(X, mode, [kh, kw], list(pads), [sh, sw], None, "NOTSET", ceil_mode, include_pad)
        assert got.shape == want.shape, (case, H, W, kh, kw, sh, sw, pads, ceil_mode)
        if mode == "max":
            np.testing.assert_array_equal(got, want.astype(np.float32))
        else:
            np.testing.assert_allclose(got, want, rtol=2e-6, atol=2e-6)
        seen_ceil_overhang += int(ceil_mode and ((H + pads[0] + pads[2] - kh) % sh or (W + pads[1] + pads[3] - kw) % sw))
    assert seen_ceil_overhang > 10   # the sweep does reach windows that hang over the end


def test_pool_against_the_library_routine():
    """torch's pooling is an independent implementation of the same definition (floor mode)."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(12)
    X = rng.standard_normal((2, 4, 9, 11)).astype(np.float32)
    t = torch.from_numpy(X)
    np.testing.assert_array_equal(ob.pool(X, "max", [3, 2], [1, 0, 1, 0], [2, 1]), F.max_pool2d(t, (3, 2), (2, 1), (1, 0)).numpy())
    for include in (0, 1):
        want = F.avg_pool2d(t, (3, 3), (2, 2), (1, 1), count_include_pad=bool(include)).numpy()
        np.testing.assert_allclose(ob.pool(X, "average", [3, 3], [1, 1, 1, 1], [2, 2], count_include_pad=include), want, rtol=2e-6, atol=2e-6)
    X1 = rng.standard_normal((3, 2, 17)).astype(np.float32)
    np.testing.assert_array_equal(ob.pool(X1, "max", [3], None, [2]), F.max_pool1d(torch.from_numpy(X1), 3, 2).numpy())


def test_pool3d_against_the_library_routine_and_the_2d_operator():
    """Three spatial axes: torch's pooling as the independent implementation (floor mode), every axis with its own extent, window,
    stride and padding; a volume of depth one must give the 2-D operator's bits; the reference's MaxPool3d shape."""
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(13)
    X = rng.standard_normal((2, 3, 7, 9, 8)).astype(np.float32)
    t = torch.from_numpy(X)
    np.testing.assert_array_equal(ob.pool(X, "max", [3, 2, 4], [1, 0, 2, 1, 0, 2], [2, 1, 3]), F.max_pool3d(t, (3, 2, 4), (2, 1, 3), (1, 0, 2)).numpy())
    for include in (0, 1):
        want = F.avg_pool3d(t, (3, 2, 2), (2, 1, 2), (1, 1, 0), count_include_pad=bool(include)).numpy()
        np.testing.assert_allclose(ob.pool(X, "average", [3, 2, 2], [1, 1, 0, 1, 1, 0], [2, 1, 2], count_include_pad=include), want, rtol=2e-6, atol=2e-6)
    want = F.max_pool3d(t, (2, 3, 2), (2, 2, 3), (0, 1, 0), ceil_mode=True).numpy()
    np.testing.assert_array_equal(ob.pool(X, "max", [2, 3, 2], [0, 1, 0, 0, 1, 0], [2, 2, 3], ceil_mode=1), want)
    X2 = rng.standard_normal((2, 3, 6, 10)).astype(np.float32)
    for mode in ("max", "average"):
        flat = ob.pool(X2, mode, [3, 2], [1, 0, 0, 1], [2, 3], count_include_pad=1)
        deep = ob.pool(X2[:, :, None], mode, [1, 3, 2], [0, 1, 0, 0, 0, 1], [1, 2, 3], count_include_pad=1)
        assert np.array_equal(deep[:, :, 0].view(np.uint32), flat.view(np.uint32))
    X3 = np.arange(27, dtype=np.float32).reshape(1, 1, 3, 3, 3)
    assert ob.pool(X3, "max", [2, 2, 2], None, [1, 1, 1]).shape == (1, 1, 2, 2, 2)
    np.testing.assert_array_equal(ob.pool(X3, "average", [3, 3, 3]).ravel(), [13.0])


def test_pool_special_cases():
    X = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    # a window that is the image is GlobalAveragePool; a 1x1 window with stride 1 is the identity
    np.testing.assert_array_equal(ob.pool(X, "average", [4, 5]), ob.global_avg_pool(X))
    np.testing.assert_array_equal(ob.pool(X, "max", [1, 1]), X)
    np.testing.assert_array_equal(ob.pool(X, "average", [1, 1]), X)
    # NaN never wins `x > value`; a window of NaNs only stays at -inf (the reference's comparison, not IEEE maximum)
    Xn = np.array([[[np.nan, 1.0, np.nan, np.nan]]], dtype=np.float32)
    np.testing.assert_array_equal(ob.pool(Xn, "max", [2], None, [2]), np.array([[[1.0, -np.inf]]], dtype=np.float32))
    # SAME_UPPER puts the odd padding sample at the end, SAME_LOWER at the beginning
    assert ob.pool_axes([5], [2], None, [1], None, "SAME_UPPER")[0][4:] == (0, 1)
    assert ob.pool_axes([5], [2], None, [1], None, "SAME_LOWER")[0][4:] == (1, 0)
    # the reference pools over the whole dilated extent: kernel 2 with dilation 2 is a dense window of 3
    np.testing.assert_array_equal(ob.pool(X, "max", [2, 2], None, [1, 1], [2, 2]), ob.pool(X, "max", [3, 3]))
    # ceil_mode with the window hanging over the end (the reference's MaxPool1d_CeilMode_Overhang shape: 6 -> 2)
    X6 = np.array([[[1, 2, 3, 4, 5, 6]]], dtype=np.float32)
    np.testing.assert_array_equal(ob.pool(X6, "max", [2], None, [3], ceil_mode=1), np.array([[[2, 5]]], dtype=np.float32))
    np.testing.assert_array_equal(ob.pool(X6, "average", [2], None, [3], ceil_mode=1), np.array([[[1.5, 4.5]]], dtype=np.float32))


def test_erf_and_elu_against_library_routines():
    from scipy import special
    x = np.linspace(-4, 4, 4001).astype(np.float32)
    np.testing.assert_allclose(ob.unary(x, 24), special.erf(x.astype(np.float64)), rtol=0, atol=2e-7)
    assert ob.unary(np.array([0.0, np.inf, -np.inf], np.float32), 24).tolist() == [0.0, 1.0, -1.0]
    elu = ob.unary_chain(x, [(23, 0.7, 0.0)])
    want = np.where(x >= 0, x, np.float32(0.7) * np.expm1(x.astype(np.float64)))
    np.testing.assert_allclose(elu, want, rtol=0, atol=2e-7)
    assert np.array_equal(elu[x >= 0], x[x >= 0])     # the positive half is the identity, bit for bit


def test_softmax_against_the_library_routine_and_its_invariants():
    from scipy import special
    rng = np.random.default_rng(31)
    for shape, axis in [((7,), 0), ((5, 11), -1), ((3, 4, 6), 1), ((2, 3, 4, 2), -2), ((4, 1000), 1), ((2, 5, 3), 0)]:
        X = (3 * rng.standard_normal(shape)).astype(np.float32)
        got = ob.softmax(X, axis)
        np.testing.assert_allclose(got, special.softmax(X.astype(np.float64), axis=axis), rtol=3e-6, atol=1e-9)
        np.testing.assert_allclose(got.sum(axis=axis), 1.0, rtol=0, atol=2e-6)
        np.testing.assert_allclose(ob.softmax(X, axis, log=True), special.log_softmax(X.astype(np.float64), axis=axis), rtol=5e-7, atol=2e-6)
        # a shift that is exact in fp32 leaves x - vmax, and with it every bit of the result, unchanged
        Xq = (np.round(X * 1024) / 1024).astype(np.float32)
        assert np.array_equal(ob.softmax(Xq, axis), ob.softmax(Xq + np.float32(8.0), axis))
    # large inputs do not overflow (the maximum is subtracted first), and a one-element axis gives exactly 1
    big = np.array([[1000.0, 999.0, -1000.0]], dtype=np.float32)
    np.testing.assert_allclose(ob.softmax(big), [[1 / (1 + np.exp(-1.0)), np.exp(-1.0) / (1 + np.exp(-1.0)), 0.0]], rtol=2e-7)
    assert ob.softmax(np.array([[3.5], [-2.0]], np.float32)).tolist() == [[1.0], [1.0]]


def test_binary_operators_against_numpy_and_the_library_semantics():
    rng = np.random.default_rng(41)
    A = (2 * rng.standard_normal((3, 1, 5, 4))).astype(np.float32)
    B = (2 * rng.standard_normal((6, 1, 4))).astype(np.float32)
    B[np.abs(B) < 0.05] = 0.5
    assert np.array_equal(ob.binary_broadcast(A, B, 0), A + B)
    assert np.array_equal(ob.binary_broadcast(A, B, 1), A - B)
    assert np.array_equal(ob.binary_broadcast(A, B, 2), A * B)
    assert np.array_equal(ob.binary_broadcast(A, B, 3), A / B)
    np.testing.assert_allclose(ob.binary_broadcast(np.abs(A) + 0.1, B, 4), np.power((np.abs(A) + 0.1).astype(np.float64), B.astype(np.float64)), rtol=3e-7)
    assert np.array_equal(ob.binary_broadcast(A, B, 5), np.maximum(A, B)) and np.array_equal(ob.binary_broadcast(A, B, 6), np.minimum(A, B))
    assert np.array_equal(ob.binary_broadcast(A, B, 7, 3.0), ((A + B) / np.float32(3.0)).astype(np.float32))
    # std::max / std::min return their FIRST argument unless the second is strictly larger / smaller (C++ [alg.min.max]):
    # a NaN in first place stays, a NaN in second place never wins, and of two zeros the first one's sign survives
    nan, one = np.array([np.nan], np.float32), np.array([1.0], np.float32)
    assert np.isnan(ob.binary_broadcast(nan, one, 5)[0]) and ob.binary_broadcast(one, nan, 5)[0] == 1.0
    assert np.isnan(ob.binary_broadcast(nan, one, 6)[0]) and ob.binary_broadcast(one, nan, 6)[0] == 1.0
    mz, pz = np.array([-0.0], np.float32), np.array([0.0], np.float32)
    assert np.signbit(ob.binary_broadcast(mz, pz, 5)[0]) and not np.signbit(ob.binary_broadcast(pz, mz, 5)[0])
    # pow special values of the C library: x^0 = 1 for any x, 1^y = 1, a negative base with a non-integer exponent is NaN
    p = ob.binary_broadcast(np.array([np.nan, 1.0, -8.0, -8.0, 0.0], np.float32), np.array([0.0, np.nan, 1.0 / 3, 2.0, -1.0], np.float32), 4)
    assert p[0] == 1.0 and p[1] == 1.0 and np.isnan(p[2]) and p[3] == 64.0 and np.isposinf(p[4])


def test_layernorm_against_the_definition():
    rng = np.random.default_rng(51)
    for shape, axis in [((3, 4), -1), ((2, 3, 4, 5), 2), ((5, 1000), 1), ((4, 6, 7), 1)]:
        X = (2 * rng.standard_normal(shape) + 0.5).astype(np.float32)
        ax = axis + len(shape) if axis < 0 else axis
        norm_shape = shape[ax:]
        scale, bias = rng.standard_normal(norm_shape).astype(np.float32), rng.standard_normal(norm_shape).astype(np.float32)
        Y, mean, inv = ob.layernorm(X, scale, bias, axis, 1e-5, stats=True)
        x64 = X.astype(np.float64).reshape(-1, int(np.prod(norm_shape)))
        m = x64.mean(axis=1, keepdims=True)
        v = ((x64 - m) ** 2).mean(axis=1, keepdims=True)
        want = (x64 - m) / np.sqrt(v + 1e-5) * scale.astype(np.float64).ravel() + bias.astype(np.float64).ravel()
        np.testing.assert_allclose(Y.reshape(want.shape), want, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(mean, m.ravel(), rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(inv, 1 / np.sqrt(v.ravel() + 1e-5), rtol=1e-5)
        # unit scale, no bias: every row comes out with zero mean and (up to epsilon) unit variance
        Z = ob.layernorm(X, np.ones(norm_shape, np.float32), None, axis, 1e-5).reshape(want.shape)
        assert np.abs(Z.mean(axis=1)).max() < 1e-5 and np.abs(Z.var(axis=1) - 1).max() < 1e-3
    # a constant row has zero variance: the output is the bias, and invStdDev is 1 / sqrt(epsilon)
    Y, mean, inv = ob.layernorm(np.full((1, 8), 3.0, np.float32), np.ones(8, np.float32), np.arange(8, dtype=np.float32), -1, 1e-4, stats=True)
    assert Y.ravel().tolist() == list(range(8)) and mean[0] == 3.0 and abs(inv[0] - 100.0) < 1e-3


def test_reduce_against_numpy_in_float64():
    rng = np.random.default_rng(77)
    np_ops = {0: lambda x, ax: x.sum(axis=ax), 1: lambda x, ax: x.mean(axis=ax), 2: lambda x, ax: (x * x).sum(axis=ax), 3: lambda x, ax: x.prod(axis=ax),
              4: lambda x, ax: np.sqrt((x * x).sum(axis=ax)), 5: lambda x, ax: x.max(axis=ax), 6: lambda x, ax: x.min(axis=ax)}
    for shape, axes in [((1, 2, 3), [1]), ((3, 4), [0]), ((2, 3, 4), [1]), ((2, 3, 4), [-1]), ((2, 3, 4, 5), [1, 2]), ((4, 512), [1]), ((5, 7), None),
                        ((6, 1, 5), [0, 2])]:
        X = rng.uniform(0.5, 1.5, shape).astype(np.float32) * rng.choice([-1.0, 1.0], shape).astype(np.float32)
        ax = tuple(range(len(shape))) if axes is None else tuple(a % len(shape) for a in axes)
        for op, f in np_ops.items():
            for keep in (0, 1):
                want = f(X.astype(np.float64), ax)
                got = ob.reduce(X, op, axes, keep)
                want = np.expand_dims(want, ax) if keep else want
                assert got.shape == np.shape(want), (shape, axes, op, keep)
                if op >= 5:
                    assert np.array_equal(got, want.astype(np.float32))
                else:
                    np.testing.assert_allclose(got, want, rtol=3e-6, atol=3e-6 * np.abs(X).sum(axis=ax).max() if op != 3 else 0)
    # the reference's own literal cases: ReduceSum {24}, ReduceSumSquare {38, 66}, ReduceMin {5, 2, 3}, ReduceMean over the first axis of iota(12) = {4, 5, 6, 7},
    # ReduceL2Large rows of r + 1 over 512 columns = (r + 1) * sqrt(512)
    x = np.array([5, 2, 3, 5, 5, 4], np.float32).reshape(1, 2, 3)
    assert ob.reduce(x, 0, [0, 1, 2], 1).ravel().tolist() == [24.0] and ob.reduce(x, 2, [2], 0).ravel().tolist() == [38.0, 66.0]
    assert ob.reduce(x, 6, [1], 0).ravel().tolist() == [5.0, 2.0, 3.0]
    assert ob.reduce(np.arange(12, dtype=np.float32).reshape(3, 4), 1, [0], 0).tolist() == [4.0, 5.0, 6.0, 7.0]
    big = np.repeat(np.arange(1, 5, dtype=np.float32)[:, None], 512, axis=1)
    np.testing.assert_allclose(ob.reduce(big, 4, [1], 0), np.arange(1, 5) * np.sqrt(512.0), rtol=1e-6)
    # empty-product and start values: a reduced length of 1 returns the element (its square, its absolute value for L2)
    one = np.array([[-3.0]], np.float32)
    assert [float(ob.reduce(one, op, [1], 0)[0]) for op in range(7)] == [-3.0, -3.0, 9.0, -3.0, 3.0, -3.0, -3.0]


def test_hard_sigmoid_hard_swish_and_swish_against_their_definitions():
    x = np.concatenate([np.linspace(-8, 8, 1601), [-3.0, 3.0, -2.5, 2.5, 0.0]]).astype(np.float32)
    x64 = x.astype(np.float64)
    hs = ob.unary_chain(x, [(R.ACT_HARDSIGMOID, 0.2, 0.5)])
    np.testing.assert_allclose(hs, np.clip(0.2 * x64 + 0.5, 0, 1), atol=1e-7)
    assert hs[x <= -2.5].max() == 0.0 and hs[x >= 2.5].min() == 1.0 and hs[-1] == 0.5       # saturates exactly; 0 -> beta
    other = ob.unary_chain(x, [(R.ACT_HARDSIGMOID, 0.5, 0.25)])                              # the attributes are used, not the defaults
    np.testing.assert_allclose(other, np.clip(0.5 * x64 + 0.25, 0, 1), atol=1e-7)
    hw = ob.unary_chain(x, [(R.ACT_HARDSWISH, 0.0, 0.0)])
    np.testing.assert_allclose(hw, x64 * np.clip(x64 / 6 + 0.5, 0, 1), rtol=2e-7, atol=2e-7)
    assert np.array_equal(hw[x >= 3], x[x >= 3]) and np.all(hw[x <= -3] == 0)                # identity above 3, zero below -3
    sw = ob.unary_chain(x, [(R.ACT_SWISH, 0.0, 0.0)])
    np.testing.assert_allclose(sw, x64 / (1 + np.exp(-x64)), rtol=3e-7, atol=1e-7)
    # Swish is x * Sigmoid(x), and Swish(x) - Swish(-x) = x
    sg = ob.unary(x, R.ACT_SIGMOID, 0.0)
    np.testing.assert_allclose(sw, x * sg, rtol=3e-7, atol=1e-7)
    np.testing.assert_allclose(sw - ob.unary_chain(-x, [(R.ACT_SWISH, 0.0, 0.0)]), x, atol=1e-6)

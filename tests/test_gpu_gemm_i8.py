"""Parity of the int8 MFMA GEMM (through the C-ABI) with the CPU oracle: bit-exact."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import util

pytestmark = pytest.mark.gpu


def run_gemm(rt, A, B, M, N, K, *, transA=0, transB=0, bias=None, scale=None, scale_scalar=1.0, q_scale=1.0,
             relu_acc=0, relu_out=0, out=0, lda=0, ldb=0, ldy=0):
    dA, dB = util.to_dev(A), util.to_dev(B)
    dbias = None if bias is None else util.to_dev(bias)
    dscale = None if scale is None else util.to_dev(scale)
    odt = {0: np.int32, 1: np.float32, 2: np.int8, 3: np.int8}[out]
    rows_y = M
    dY = util.dev_empty((rows_y, ldy or N), odt)
    dY.fill_(0)
    d = R.GemmI8Desc()
    d.M, d.N, d.K, d.transA, d.transB = M, N, K, transA, transB
    d.lda, d.ldb, d.ldy = lda, ldb, ldy
    d.A, d.B, d.bias, d.scale = util.ptr(dA), util.ptr(dB), util.ptr(dbias), util.ptr(dscale)
    d.scale_scalar, d.q_scale = scale_scalar, q_scale
    d.relu_acc, d.relu_out, d.out = relu_acc, relu_out, out
    d.Y = util.ptr(dY)
    need = rt.lib.sofie_hip_gemm_i8_workspace(C.byref(d))
    ws = util.dev_empty((max(need, 256),), np.int8)
    d.workspace, d.workspace_bytes = util.ptr(ws), need
    import torch
    torch.cuda.synchronize()
    print("gemm_i8 M=%d N=%d K=%d tA=%d tB=%d out=%d" % (M, N, K, transA, transB, out), flush=True)
    rt.call("sofie_hip_gemm_i8", C.byref(d))
    rt.sync()
    return util.to_host(dY)[:, :N]


SHAPES = [(1, 1, 1), (32, 32, 32), (64, 64, 64), (33, 65, 47), (100, 200, 300), (257, 255, 129), (128, 128, 16),
          (256, 256, 256), (300, 520, 1024), (512, 1024, 768), (17, 4096, 64), (1024, 1024, 1024)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_int32_accumulate_matches_oracle(rt, M, N, K):
    A = util.int8_sym(3001 + M, M * K).reshape(M, K)
    Bt = util.int8_sym(3002 + N, N * K).reshape(N, K)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, out=R.I8OUT_I32)
    want = ob.matmul_integer(A, Bt, M=M, N=N, K=K, transB=1, omp=True)
    assert np.array_equal(got, want)
    # numpy int64 as a second arbiter
    assert np.array_equal(got, (A.astype(np.int64) @ Bt.astype(np.int64).T).astype(np.int32))


@pytest.mark.parametrize("tile", [64, 128, 256, 258])     # 258: the 256 x 128 tile that shares a CU with a second workgroup
@pytest.mark.parametrize("M,N,K", [(300, 520, 1024), (96, 160, 80), (513, 257, 2048 + 48)])
def test_every_tile_configuration(rt, opt, tile, M, N, K):
    A = util.int8_sym(11, M * K).reshape(M, K)
    Bt = util.int8_sym(12, N * K).reshape(N, K)
    opt("i8_tile", tile)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, out=R.I8OUT_I32)
    assert np.array_equal(got, ob.matmul_integer(A, Bt, M=M, N=N, K=K, transB=1, omp=True))


@pytest.mark.parametrize("transA,transB", [(0, 0), (1, 0), (1, 1)])
def test_onnx_layouts_go_through_the_workspace(rt, transA, transB):
    M, N, K = 130, 77, 200
    A = util.int8_sym(21, M * K).reshape((K, M) if transA else (M, K))
    B = util.int8_sym(22, N * K).reshape((N, K) if transB else (K, N))
    got = run_gemm(rt, A, B, M, N, K, transA=transA, transB=transB, out=R.I8OUT_I32)
    assert np.array_equal(got, ob.matmul_integer(A, B, M=M, N=N, K=K, transA=transA, transB=transB))


@pytest.mark.parametrize("out,relu_acc,relu_out", [(R.I8OUT_F32, 0, 0), (R.I8OUT_F32, 1, 0), (R.I8OUT_I8, 0, 0),
                                                   (R.I8OUT_I8, 0, 1), (R.I8OUT_I8_DQQ, 1, 0), (R.I8OUT_I32, 1, 0)])
@pytest.mark.parametrize("M,N,K", [(200, 136, 512), (64, 50, 1000)])
def test_fused_epilogues_bit_exact(rt, out, relu_acc, relu_out, M, N, K):
    A = util.int8_sym(31, M * K).reshape(M, K)
    Bt = util.int8_sym(32, N * K).reshape(N, K)
    bias = util.int32_range(33, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(34, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    kw = dict(bias=bias, scale=scale, q_scale=np.float32(0.037), relu_acc=relu_acc, relu_out=relu_out, out=out)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, **kw)
    want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, **kw)
    assert got.dtype == want.dtype
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    if out == R.I8OUT_I8:
        assert got.min() <= (0 if relu_out else -100) and got.max() >= 100  # the data really spans the int8 range


def _f32_from_bits(b):
    return np.array([b], dtype=np.uint32).view(np.float32)[0]


@pytest.mark.parametrize("q", [3.0, 0.037, 0.601829112, 16.3691254, -7.25, float(_f32_from_bits(0x3fffffff)), 2.0 ** -31])
@pytest.mark.parametrize("M,N,K", [(256, 384, 512), (200, 136, 512), (64, 50, 1000)])
def test_dequantize_quantize_with_a_per_tensor_scale(rt, q, M, N, K):
    """With a per-tensor scale the runtime may form the quotient of SOFIE_I8OUT_I8_DQQ from the reciprocal of q_scale; the
    last two divisors (significand all ones, out of range) keep the division.  Either way the bytes are those of
    sat8(rne(fl(fl(acc * s) / q))) in IEEE fp32, here from numpy's division.  s = q / 2 puts every odd accumulator on a tie."""
    A = util.int8_sym(51, M * K).reshape(M, K)
    Bt = util.int8_sym(52, N * K).reshape(N, K)
    acc = ob.matmul_integer(A, Bt, M=M, N=N, K=K, transB=1)
    q = np.float32(q)
    spread = np.float32(np.abs(acc).max())
    for s in (np.float32(abs(q) * 127.0 / spread), np.float32(abs(q) * 300.0 / spread), np.float32(abs(q) / 2)):
        got = run_gemm(rt, A, Bt, M, N, K, transB=1, scale_scalar=s, q_scale=q, out=R.I8OUT_I8_DQQ)
        v = (acc.astype(np.float32) * s).astype(np.float32)
        want = np.clip(np.rint((v / q).astype(np.float32)), -128, 127).astype(np.int8)
        assert np.array_equal(got, want), (float(q), float(s))
        assert np.array_equal(got, ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, scale_scalar=s, q_scale=q, out=R.I8OUT_I8_DQQ))
    assert got.min() == -128 and got.max() == 127


def test_per_tensor_scale_and_odd_leading_dimensions(rt):
    M, N, K = 70, 90, 160
    lda, ldb, ldy = 176, 192, 101
    A = util.int8_sym(41, M * lda).reshape(M, lda)
    Bt = util.int8_sym(42, N * ldb).reshape(N, ldb)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, lda=lda, ldb=ldb, ldy=ldy, scale_scalar=np.float32(1e-3), out=R.I8OUT_I8)
    want = ob.gemm_i8(np.ascontiguousarray(A[:, :K]), np.ascontiguousarray(Bt[:, :K]), M=M, N=N, K=K, transB=1,
                      scale_scalar=np.float32(1e-3), out=R.I8OUT_I8)
    assert np.array_equal(got, want)


def test_round_half_even_and_saturation(rt):
    # K = 1: acc = a*b exactly; scale 0.5 puts odd products on .5 ties
    a = np.array([[1], [3], [5], [-1], [-3], [127], [-127], [127], [-128], [0]], dtype=np.int8)
    bt = np.array([[1], [2], [127], [-127], [51]], dtype=np.int8)
    M, N = a.shape[0], bt.shape[0]
    got = run_gemm(rt, a, bt, M, N, 1, transB=1, scale_scalar=np.float32(0.5), out=R.I8OUT_I8)
    acc = a.astype(np.int64) @ bt.astype(np.int64).T
    want = np.clip(np.round(acc * 0.5), -128, 127).astype(np.int8)  # numpy rounds half to even
    assert np.array_equal(got, want)
    assert got[0, 0] == 0 and got[1, 0] == 2 and got[2, 0] == 2 and got[3, 0] == 0 and got[4, 0] == -2
    assert got[5, 2] == 127 and got[6, 2] == -128  # saturation
    assert np.array_equal(got, ob.gemm_i8(a, bt, M=M, N=N, K=1, transB=1, scale_scalar=np.float32(0.5), out=R.I8OUT_I8))


def test_empty_dimensions(rt):
    d = R.GemmI8Desc()
    d.M, d.N, d.K = 0, 16, 16
    rt.call("sofie_hip_gemm_i8", C.byref(d))
    # K = 0: the dot product is empty, the output is the epilogue of 0 (+ bias)
    bias = np.arange(-3, 5, dtype=np.int32)
    got = run_gemm(rt, np.zeros((4, 1), np.int8), np.zeros((8, 1), np.int8), 4, 8, 0, transB=1, bias=bias, out=R.I8OUT_I32)
    assert np.array_equal(got, np.tile(bias, (4, 1)))


def test_bad_arguments_are_refused(rt):
    from sofie_amd import SofieHipError
    d = R.GemmI8Desc()
    d.M, d.N, d.K = 16, 16, 16
    with pytest.raises(SofieHipError, match="Y is NULL"):
        rt.call("sofie_hip_gemm_i8", C.byref(d))
    y = util.dev_empty((16, 16), np.int32)
    a = util.to_dev(np.zeros((16, 16), np.int8))
    d.Y, d.A, d.B = util.ptr(y), util.ptr(a), util.ptr(a)
    with pytest.raises(SofieHipError, match="workspace"):
        rt.call("sofie_hip_gemm_i8", C.byref(d))  # B is [K,N] and no workspace was given
    d.transB, d.out = 1, 7
    with pytest.raises(SofieHipError, match="unknown output kind"):
        rt.call("sofie_hip_gemm_i8", C.byref(d))


def test_full_size_8192_sampled_rows_and_linearity(rt):
    """benchmark configuration 3 at M=N=K=8192: full rows checked bit-exactly against the oracle on a sample,
    plus a size-independent property: G(A1) + G(A2) == G(A1 + A2) for int32 outputs."""
    import torch
    M = N = K = 8192
    A = util.int8_sym(3001, M * K).reshape(M, K)
    Bt = util.int8_sym(3002, N * K).reshape(N, K)
    bias = util.int32_range(3003, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(3004, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, bias=bias, scale=scale, relu_out=1, out=R.I8OUT_I8)
    rows = np.array([0, 1, 31, 32, 255, 256, 4095, 4096, 5000, 8190, 8191, 777])
    want = ob.gemm_i8(np.ascontiguousarray(A[rows]), Bt, M=len(rows), N=N, K=K, transB=1, omp=True, bias=bias, scale=scale,
                      relu_out=1, out=R.I8OUT_I8)
    assert np.array_equal(got[rows], want)
    cols = np.array([0, 5, 63, 64, 4097, 8191])
    want_c = ob.gemm_i8(A, np.ascontiguousarray(Bt[cols]), M=M, N=len(cols), K=K, transB=1, omp=True, bias=bias[cols],
                        scale=scale[cols], relu_out=1, out=R.I8OUT_I8)
    assert np.array_equal(got[:, cols], want_c)
    assert got.max() == 127 and (got == 0).mean() > 0.3
    del got
    # linearity on halves of the value range (no int8 overflow in A1 + A2)
    A1 = (A >> 1).astype(np.int8)
    A2 = (A - A1).astype(np.int8)
    g = run_gemm(rt, A, Bt, M, N, K, transB=1, out=R.I8OUT_I32)
    g1 = run_gemm(rt, A1, Bt, M, N, K, transB=1, out=R.I8OUT_I32)
    g2 = run_gemm(rt, A2, Bt, M, N, K, transB=1, out=R.I8OUT_I32)
    assert np.array_equal(g, g1 + g2)
    torch.cuda.empty_cache()


def test_short_reduction_over_many_tiles_takes_the_shared_cu_tile(rt):
    """K <= 1024 with at least 512 tiles of 256 x 128: the heuristic's own choice of the two-per-CU tile (ragged M and N)."""
    M, N, K = 8192 + 37, 2048 + 5, 512
    A = util.int8_sym(13, M * K).reshape(M, K)
    Bt = util.int8_sym(14, N * K).reshape(N, K)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, out=R.I8OUT_I32)
    assert np.array_equal(got, ob.matmul_integer(A, Bt, M=M, N=N, K=K, transB=1, omp=True))


@pytest.mark.parametrize("out,relu_acc,relu_out", [(R.I8OUT_I32, 0, 0), (R.I8OUT_F32, 1, 0), (R.I8OUT_I8, 0, 1), (R.I8OUT_I8, 0, 0),
                                                   (R.I8OUT_I8_DQQ, 1, 0)])
@pytest.mark.parametrize("M,N,K", [(256, 256, 384), (512, 768, 512), (1280, 512, 1152), (256, 4352, 640)])
def test_persistent_kernel_forced_on_small_shapes(rt, opt, out, relu_acc, relu_out, M, N, K):
    """Tile 512 asks for the persistent 256 x 256 kernel (eight waves, tile store from registers) where the heuristic would
    not pick it: one tile, fewer tiles than CUs, more tiles than CUs (17 x 1 and 5 x 2 lists of uneven length per workgroup
    do not occur at these sizes, so the 4352-column case gives workgroups 0..16 one tile each), K of 3, 4, 5 and 9 slab pairs."""
    A = util.int8_sym(51 + M, M * K).reshape(M, K)
    Bt = util.int8_sym(52 + N, N * K).reshape(N, K)
    bias = util.int32_range(53, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(54, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    kw = dict(bias=bias, scale=scale, q_scale=np.float32(0.041), relu_acc=relu_acc, relu_out=relu_out, out=out)
    opt("i8_tile", 512)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, **kw)
    want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, omp=True, **kw)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("out,relu_acc,relu_out,M,N,K", [(R.I8OUT_I8, 0, 1, 300, 528, 384), (R.I8OUT_I8, 0, 0, 1000, 272, 512), (R.I8OUT_I8_DQQ, 1, 0, 257, 256, 640),
                                                         (R.I8OUT_I32, 0, 0, 260, 516, 384), (R.I8OUT_F32, 1, 0, 511, 260, 384),
                                                         (R.I8OUT_I8, 0, 1, 2000, 8208, 512)])
def test_persistent_kernel_on_sizes_that_are_not_multiples_of_its_tile(rt, opt, out, relu_acc, relu_out, M, N, K):
    """M and N that do not divide into 256 x 256 tiles: the last tile of a row / column of tiles is moved back to end at the edge
    and overlaps its neighbour (both store the shared outputs, with the same values).  N must keep the moved tile on a 16-byte
    boundary of the output rows (16 elements for 1-byte outputs, 4 for 4-byte ones).  2000 x 8208: 8 x 33 = 264 tiles, more
    than compute units, by the heuristic's own choice; the others are forced."""
    A = util.int8_sym(91 + M, M * K).reshape(M, K)
    Bt = util.int8_sym(92 + N, N * K).reshape(N, K)
    bias = util.int32_range(93, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(94, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    kw = dict(bias=bias, scale=scale, q_scale=np.float32(0.041), relu_acc=relu_acc, relu_out=relu_out, out=out)
    if M < 2000:
        opt("i8_tile", 512)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, **kw)
    want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, omp=True, **kw)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("tile", [0, 64, 512])
@pytest.mark.parametrize("out,relu_acc,relu_out", [(R.I8OUT_I8, 0, 0), (R.I8OUT_I8, 0, 1), (R.I8OUT_I8, 1, 0), (R.I8OUT_I8_DQQ, 0, 0),
                                                   (R.I8OUT_I8_DQQ, 1, 0), (R.I8OUT_F32, 0, 1), (R.I8OUT_F32, 0, 0)])
def test_scales_that_are_negative_zero_huge_or_not_numbers(rt, opt, tile, out, relu_acc, relu_out):
    """Per-channel scales the conversions have short cuts around: negative, +-0, subnormal, the largest float, +-infinity and
    NaN, next to ordinary ones.  The 1-byte stores must give the oracle's bytes (a NaN product is stored as 0, an infinite one
    saturates), the fp32 store its values (NaN where the oracle has NaN).  Tile 0: the heuristic's kernel (store through LDS),
    64: the small tile, 512: the persistent kernel (store from registers)."""
    M, N, K = 256, 512, 384
    A = util.int8_sym(71, M * K).reshape(M, K)
    A[5, :] = 0                                   # a row of zero accumulators: 0 * inf is NaN
    Bt = util.int8_sym(72, N * K).reshape(N, K)
    scale = ((0.5 + util.uniform01(73, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    special = [-1e-3, -0.0, 0.0, 1e-42, -1e-42, 3.4028235e38, -3.4028235e38, np.inf, -np.inf, np.nan, 1e30, -7.0]
    for k, v in enumerate(special):
        scale[3 + 17 * k] = np.float32(v)
        scale[260 + 11 * k] = np.float32(v)
    bias = util.int32_range(74, N, -(1 << 12), 1 << 12)
    kw = dict(bias=bias, scale=scale, q_scale=np.float32(0.37), relu_acc=relu_acc, relu_out=relu_out, out=out)
    opt("i8_tile", tile)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, **kw)
    with np.errstate(all="ignore"):
        want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, **kw)
    if out == R.I8OUT_F32:
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    else:
        assert np.array_equal(got, want), np.argwhere(got != want)[:8]


@pytest.mark.parametrize("tile", [0, 512])
def test_dequantize_quantize_with_a_huge_output_scale_and_infinite_channel_scales(rt, opt, tile):
    """SOFIE_I8OUT_I8_DQQ with q_scale near the top of the float range: (acc * inf) / q_scale saturates, (acc * FLT_MAX) /
    q_scale does not.  The store from registers, which replaces an infinite scale by FLT_MAX, must not be given this product
    (tile 512 asks for it; the library has to decline and take a kernel with the exact conversion)."""
    M, N, K = 256, 256, 384
    A = util.int8_sym(81, M * K).reshape(M, K)
    A[7, :] = 0
    A[9, :] = 0
    A[9, 0] = 1                                   # accumulators of +-1 .. +-127: the smallest non-zero products
    Bt = util.int8_sym(82, N * K).reshape(N, K)
    scale = np.full(N, np.float32(1e-3), np.float32)
    scale[::3] = np.inf
    scale[1::7] = -np.inf
    scale[2::11] = np.float32(3.4028235e38)
    kw = dict(scale=scale, q_scale=np.float32(3e37), relu_acc=0, relu_out=0, out=R.I8OUT_I8_DQQ)
    opt("i8_tile", tile)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, **kw)
    with np.errstate(all="ignore"):
        want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, **kw)
    assert np.array_equal(got, want), np.argwhere(got != want)[:8]


def test_config3_at_1024_int8_output_in_full(rt):
    """benchmark configuration 3 at M=N=K=1024 with its own epilogue (per-channel scale, bias, relu, int8 out): every element."""
    M = N = K = 1024
    A = util.int8_sym(3001, M * K).reshape(M, K)
    Bt = util.int8_sym(3002, N * K).reshape(N, K)
    bias = util.int32_range(3003, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(3004, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    kw = dict(bias=bias, scale=scale, relu_out=1, out=R.I8OUT_I8)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, **kw)
    want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, omp=True, **kw)
    assert np.array_equal(got, want)
    assert got.max() == 127 and (got == 0).mean() > 0.3


def test_config3_at_4096_sampled_rows_and_columns(rt):
    """benchmark configuration 3 at M=N=K=4096 (one 256 x 256 tile per compute unit: no workgroup takes a second tile, and
    the loads that run past the end of each one-tile list are the filler path): sampled full rows and columns, bit-exact."""
    M = N = K = 4096
    A = util.int8_sym(3001, M * K).reshape(M, K)
    Bt = util.int8_sym(3002, N * K).reshape(N, K)
    bias = util.int32_range(3003, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(3004, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, bias=bias, scale=scale, relu_out=1, out=R.I8OUT_I8)
    rows = np.array([0, 1, 15, 16, 127, 128, 255, 256, 2047, 2048, 3000, 4094, 4095])
    want = ob.gemm_i8(np.ascontiguousarray(A[rows]), Bt, M=len(rows), N=N, K=K, transB=1, omp=True, bias=bias, scale=scale,
                      relu_out=1, out=R.I8OUT_I8)
    assert np.array_equal(got[rows], want)
    cols = np.array([0, 3, 4, 63, 64, 255, 256, 2049, 4095])
    want_c = ob.gemm_i8(A, np.ascontiguousarray(Bt[cols]), M=M, N=len(cols), K=K, transB=1, omp=True, bias=bias[cols],
                        scale=scale[cols], relu_out=1, out=R.I8OUT_I8)
    assert np.array_equal(got[:, cols], want_c)
    assert got.max() == 127 and (got == 0).mean() > 0.3


def test_persistent_kernel_more_tiles_than_cus(rt):
    """2304 x 8192: 9 x 32 = 288 tiles on 256 CUs, so 32 workgroups take a second tile and the loads of the others run past
    the end of their lists; per-tensor scale (no bias, no scale vector)."""
    M, N, K = 2304, 8192, 512
    A = util.int8_sym(61, M * K).reshape(M, K)
    Bt = util.int8_sym(62, N * K).reshape(N, K)
    got = run_gemm(rt, A, Bt, M, N, K, transB=1, scale_scalar=np.float32(3e-4), out=R.I8OUT_I8)
    want = ob.gemm_i8(A, Bt, M=M, N=N, K=K, transB=1, omp=True, scale_scalar=np.float32(3e-4), out=R.I8OUT_I8)
    assert np.array_equal(got, want)

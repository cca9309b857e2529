"""sofie_hip_gemm_i8_noalloc (static device scratch, no allocation) against sofie_hip_gemm_i8 on the same descriptor: the same
bits, on two calls in a row of which the second is smaller (the scratch keeps the first call's contents)."""
import ctypes as C

import numpy as np
import pytest

from sofie_amd import runtime as R, SofieHipError
from tests import util

pytestmark = pytest.mark.gpu


def both(rt, A, B, M, N, K, transA, transB, **epi):
    """Runs the descriptor through the allocation-free entry point (no workspace in the descriptor) and through
    sofie_hip_gemm_i8 (workspace from the caller); returns the two outputs."""
    import torch
    dA, dB = util.to_dev(A), util.to_dev(B)
    bias, scale = epi.get("bias"), epi.get("scale")
    dbias = None if bias is None else util.to_dev(bias)
    dscale = None if scale is None else util.to_dev(scale)
    out = epi.get("out", R.I8OUT_I32)
    odt = {0: np.int32, 1: np.float32, 2: np.int8, 3: np.int8}[out]
    outs = []
    for entry in ("sofie_hip_gemm_i8_noalloc", "sofie_hip_gemm_i8"):
        dY = util.dev_empty((M, N), odt)
        dY.fill_(0)
        d = R.GemmI8Desc()
        d.M, d.N, d.K, d.transA, d.transB = M, N, K, transA, transB
        d.A, d.B, d.bias, d.scale = util.ptr(dA), util.ptr(dB), util.ptr(dbias), util.ptr(dscale)
        d.scale_scalar, d.q_scale = epi.get("scale_scalar", 1.0), epi.get("q_scale", 1.0)
        d.relu_acc, d.relu_out, d.out = epi.get("relu_acc", 0), epi.get("relu_out", 0), out
        d.Y = util.ptr(dY)
        ws = None
        if entry == "sofie_hip_gemm_i8":
            need = rt.lib.sofie_hip_gemm_i8_workspace(C.byref(d))
            ws = util.dev_empty((max(need, 256),), np.int8)
            d.workspace, d.workspace_bytes = util.ptr(ws), need
        torch.cuda.synchronize()
        print(entry, M, N, K, transA, transB, out, flush=True)
        rt.call(entry, C.byref(d))
        rt.sync()
        outs.append(util.to_host(dY))
    return outs


def test_no_alloc_entry_point_matches_the_workspace_one_on_two_calls_in_a_row(rt):
    # first call: both operands need the re-layout (A stored [K,M], B stored [K,N]): 2 x 640 KB of scratch
    M, N, K = 700, 900, 1024
    A = util.int8_sym(7001, K * M).reshape(K, M)
    B = util.int8_sym(7002, K * N).reshape(K, N)
    bias = util.int32_range(7003, N, -(1 << 15), 1 << 15)
    scale = ((0.5 + util.uniform01(7004, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32)
    got, want = both(rt, A, B, M, N, K, 1, 0, bias=bias, scale=scale, relu_out=1, out=R.I8OUT_I8)
    assert np.array_equal(got, want) and got.max() > 50
    # second call, smaller, other shapes: the scratch still holds the first call's operands beyond what this one overwrites
    M, N, K = 130, 77, 200
    A = util.int8_sym(7011, M * K).reshape(M, K)
    B = util.int8_sym(7012, K * N).reshape(K, N)
    got, want = both(rt, A, B, M, N, K, 0, 0, out=R.I8OUT_I32)
    assert np.array_equal(got, want)
    assert np.array_equal(got, (A.astype(np.int64) @ B.astype(np.int64)).astype(np.int32))
    # operands that need no re-layout use no scratch at all
    Bt = np.ascontiguousarray(B.T)
    got, want = both(rt, A, Bt, M, N, K, 0, 1, scale_scalar=np.float32(2e-4), out=R.I8OUT_F32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_no_alloc_entry_point_refuses_what_does_not_fit(rt):
    # B [K,N] of 16 MiB: twice the static buffer
    K, N, M = 4096, 4096, 16
    dA = util.to_dev(np.zeros((M, K), np.int8))
    dB = util.to_dev(np.zeros((K, N), np.int8))
    dY = util.dev_empty((M, N), np.int32)
    d = R.GemmI8Desc()
    d.M, d.N, d.K, d.transA, d.transB = M, N, K, 0, 0
    d.A, d.B, d.Y, d.out = util.ptr(dA), util.ptr(dB), util.ptr(dY), R.I8OUT_I32
    with pytest.raises(SofieHipError, match="static buffer holds"):
        rt.call("sofie_hip_gemm_i8_noalloc", C.byref(d))

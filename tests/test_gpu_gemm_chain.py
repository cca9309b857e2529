"""sofie_hip_gemm_chain_f32: a sequence of products in which each reads what the one before wrote, as one launch at small
batch.  Every layer's output is compared with the CPU restatement of the reference's Gemm + activation run layer by layer:
|got - want| <= 1e-5 * (|want| + sum_k |a_k b_k|), the bound of the single product (the summation order is free)."""
import ctypes as C

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import util

pytestmark = pytest.mark.gpu


def run_chain(rt, X, layers, alias=None):
    """layers: dicts with W (stored as given), transB, bias (or None), bias_mode, act, act_alpha, alpha, post (list or None),
    residual (array of the output's shape or None).  alias = {l: m}: layer l writes into the buffer of layer m < l (same
    size, or the first floats of it when the shapes differ).  Returns the device results of every layer."""
    n = len(layers)
    descs = (R.GemmF32Desc * n)()
    keep, outs = [], []
    dA = util.to_dev(X)
    M, K = X.shape
    for l, L in enumerate(layers):
        N = L["W"].shape[0] if L["transB"] else L["W"].shape[1]
        dW = util.to_dev(L["W"])
        dC = None if L.get("bias") is None else util.to_dev(L["bias"])
        dR = None if L.get("residual") is None else util.to_dev(L["residual"])
        if alias and l in alias:
            dY = outs[alias[l]]
            if tuple(dY.shape) != (M, N):      # another shape: the first M * N floats of that buffer
                dY = dY.view(-1)[:M * N].view(M, N)
        else:
            dY = util.dev_empty((M, N), np.float32)
        d = descs[l]
        d.M, d.N, d.K, d.transA, d.transB = M, N, K, 0, int(L["transB"])
        d.alpha, d.beta, d.batch = L.get("alpha", 1.0), L.get("beta", 1.0), 1
        d.A, d.B, d.C, d.Y = util.ptr(dA), util.ptr(dW), util.ptr(dC), util.ptr(dY)
        d.bias_mode, d.act, d.act_alpha = L.get("bias_mode", R.BIAS_NONE if dC is None else R.BIAS_ROW), L.get("act", 0), L.get("act_alpha", 0.0)
        if L.get("post"):
            post = R.PostOps.of(L["post"])
            keep.append(post)
            d.post = C.pointer(post)
        d.residual = util.ptr(dR)
        keep += [dW, dC, dR, dA]
        outs.append(dY)
        dA, K = dY, N
    import torch
    torch.cuda.synchronize()
    rt.call("sofie_hip_gemm_chain_f32", descs, n)
    rt.sync()
    return [util.to_host(y) for y in outs]


def oracle_chain(X, layers):
    """Layer by layer on the CPU, each layer fed the ORACLE's previous output; returns outputs and the magnitudes sum|a b|."""
    outs, mags = [], []
    A = X
    for L in layers:
        W = L["W"]
        M, K = A.shape
        N = W.shape[0] if L["transB"] else W.shape[1]
        bm = L.get("bias_mode", R.BIAS_NONE if L.get("bias") is None else R.BIAS_ROW)
        y = ob.gemm_f32(A, W, L.get("bias"), M=M, N=N, K=K, transB=int(L["transB"]), alpha=L.get("alpha", 1.0), beta=L.get("beta", 1.0), bias_mode=bm, act=0)
        if L.get("residual") is not None:
            y = (y + L["residual"]).astype(np.float32)
        ops = ([(L["act"], L.get("act_alpha", 0.0), 0.0)] if L.get("act", 0) else []) + list(L.get("post") or [])
        if ops:
            y = ob.unary_chain(y, ops)
        Wm = W.T if L["transB"] else W
        mags.append(abs(L.get("alpha", 1.0)) * (np.abs(A).astype(np.float64) @ np.abs(Wm).astype(np.float64)))
        outs.append(y)
        A = y
    return outs, mags


def check(got, want, mags):
    # an error of layer l-1 within its bound moves layer l by at most that bound times sum|w| -- small against this
    # layer's own bound for these contracting activations; the allowance grows with the layer
    for l, (g, w, m) in enumerate(zip(got, want, mags)):
        assert g.shape == w.shape
        err = np.abs(g.astype(np.float64) - w)
        assert np.all(err <= 1e-5 * (l + 1) * (np.abs(w) + m) + 1e-30), (l, err.max())
        assert w.std() > 1e-3


def mlp_layers(dims, seed, transB=True, act=R.ACT_RELU):
    layers = []
    for l in range(len(dims) - 1):
        K, N = dims[l], dims[l + 1]
        W = util.normal(seed + 10 * l, K * N, 1.0 / np.sqrt(K)).reshape((N, K) if transB else (K, N))
        layers.append(dict(W=W, transB=transB, bias=util.normal(seed + 10 * l + 1, N, 0.1), act=act if l < len(dims) - 2 else 0))
    return layers


@pytest.mark.parametrize("M", [1, 5, 64, 100, 200, 256, 300])
@pytest.mark.parametrize("transB", [True, False])
def test_the_benchmark_mlp_as_a_chain(rt, M, transB):
    """784 -> 128 -> 64 -> 10 with Relu between the layers; 300 rows are past the one-launch limit and run layer by layer."""
    X = util.uniform01(900 + M, M * 784).reshape(M, 784)
    layers = mlp_layers([784, 128, 64, 10], 910, transB)
    print("gemm chain", M, transB, flush=True)
    got = run_chain(rt, X, layers)
    want, mags = oracle_chain(X, layers)
    check(got, want, mags)


@pytest.mark.parametrize("fused", ["0", "1"])
def test_chain_with_every_epilogue_feature(rt, fused, opt):
    """Odd widths, both weight layouts, alpha, every bias mode, an activation with a chain behind it, a residual: the one-launch
    form and the layer-by-layer form of the same call agree with the oracle."""
    opt("f32_chain", int(fused))
    M = 37
    X = util.normal(930, M * 50).reshape(M, 50)
    layers = [
        dict(W=util.normal(931, 50 * 77, 0.15).reshape(77, 50), transB=True, bias=util.normal(932, 77), act=R.ACT_TANH, alpha=0.7),
        dict(W=util.normal(933, 77 * 301, 0.1).reshape(77, 301), transB=False, bias=util.normal(934, M), bias_mode=R.BIAS_COL, act=R.ACT_LEAKYRELU,
             act_alpha=0.2, post=[(R.ACT_SIGMOID, 0, 0), (R.ACT_CLIP, 0.1, 0.9)]),
        dict(W=util.normal(935, 301 * 9, 0.1).reshape(9, 301), transB=True, bias=util.normal(936, 1), bias_mode=R.BIAS_SCALAR,
             residual=util.normal(937, M * 9).reshape(M, 9), act=R.ACT_RELU),
        dict(W=util.normal(938, 9 * 33, 0.3).reshape(9, 33), transB=False, bias=util.normal(939, M * 33).reshape(M, 33), bias_mode=R.BIAS_FULL, beta=0.5),
        dict(W=util.normal(940, 33 * 2, 0.3).reshape(2, 33), transB=True, bias=None, act=R.ACT_GELU),
    ]
    print("gemm chain features, fused =", fused, flush=True)
    got = run_chain(rt, X, layers)
    want, mags = oracle_chain(X, layers)
    check(got, want, mags)


def test_layers_that_share_memory_run_layer_by_layer(rt):
    """A caller that planned the chain's tensors by per-layer lifetimes hands layer 2 the buffer of layer 0 (dead once layer 1 has
    read it).  In one launch a workgroup's layer-0 rows would land on rows of layer 2 that another workgroup has finished; the
    entry point sees the overlap and launches per layer, so layers 1 and 2 come out right."""
    M = 64
    X = util.normal(960, M * 32).reshape(M, 32)
    layers = mlp_layers([32, 128, 64, 128], 961, act=R.ACT_TANH)
    got = run_chain(rt, X, layers, alias={2: 0})
    want, mags = oracle_chain(X, layers)
    check(got[1:], want[1:], mags[1:])
    assert np.array_equal(got[0], got[2])  # the shared buffer holds layer 2's result


@pytest.mark.parametrize("fused", [-1, 1])
def test_layers_that_share_memory_in_another_shape_run_layer_by_layer(rt, opt, fused):
    """Layer 2 (64 columns) written into the first half of the buffer of layer 0 (128 columns): the rows of the two tensors do not
    coincide, so one launch would let a workgroup's layer-2 rows overwrite layer-0 rows that another workgroup still has to
    read.  The entry point must launch layer by layer, by its own choice (-1) and when the one-launch form is asked for (1)."""
    opt("f32_chain", fused)
    M = 64
    X = util.normal(970, M * 32).reshape(M, 32)
    layers = mlp_layers([32, 128, 64, 64], 971, act=R.ACT_TANH)
    got = run_chain(rt, X, layers, alias={2: 0})
    want, mags = oracle_chain(X, layers)
    check(got[1:], want[1:], mags[1:])


def test_chain_of_one_wide_rows_and_refusals(rt):
    # a single layer is the plain product; rows of 3000 floats at 200 rows (4 rows per workgroup) exceed LDS: layer by layer
    X = util.normal(950, 200 * 3000).reshape(200, 3000)
    layers = mlp_layers([3000, 40, 12], 951)
    got = run_chain(rt, X, layers)
    want, mags = oracle_chain(X, layers)
    check(got, want, mags)
    got = run_chain(rt, X[:3], layers[:1])
    want, mags = oracle_chain(X[:3], layers[:1])
    check(got, want, mags)
    # a layer that does not read its predecessor's output is refused before anything runs
    descs = (R.GemmF32Desc * 2)()
    x = util.to_dev(np.zeros((4, 4), np.float32))
    for d in descs:
        d.M = d.N = d.K = 4
        d.batch, d.alpha = 1, 1.0
        d.A = d.B = d.Y = util.ptr(x)
    y2 = util.to_dev(np.zeros((4, 4), np.float32))
    descs[0].Y = util.ptr(y2)
    descs[1].A = util.ptr(x)
    with pytest.raises(R.SofieHipError, match="does not read the output"):
        rt.call("sofie_hip_gemm_chain_f32", descs, 2)
    with pytest.raises(R.SofieHipError, match="layers"):
        rt.call("sofie_hip_gemm_chain_f32", descs, 17)

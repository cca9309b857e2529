"""numpy/ctypes view of the CPU oracle (oracle/sofie_oracle.c).  TEST INFRASTRUCTURE.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module; the
product path (sofie_amd/) never does.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_libs = {}


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def load(omp=False):
    name = "libsofie_oracle_omp.so" if omp else "libsofie_oracle.so"
    if name not in _libs:
        path = os.path.join(_HERE, name)
        if not os.path.exists(path):
            raise RuntimeError("%s is not built: run `make -C oracle`" % path)
        lib = C.CDLL(path)
        lib.oracle_e4m3_to_f32.restype = C.c_float
        lib.oracle_e4m3_to_f32.argtypes = [C.c_uint8]
        lib.oracle_f32_to_e4m3.restype = C.c_uint8
        lib.oracle_f32_to_e4m3.argtypes = [C.c_float]
        lib.oracle_f32_to_bf16.restype = C.c_uint16
        lib.oracle_f32_to_bf16.argtypes = [C.c_float]
        lib.oracle_num_threads.restype = C.c_int
        _libs[name] = lib
    return _libs[name]


def load_ref_planner():
    """The reference's own OrganizeMemory (oracle/_ref), or None where it was not built."""
    path = os.path.join(_HERE, "_ref", "libref_planner.so")
    if not os.path.exists(path):
        return None
    return C.CDLL(path)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def gemm_f32(A, B, C_=None, *, M, N, K, transA=0, transB=0, alpha=1.0, beta=1.0, bias_mode=0, act=0, act_alpha=0.0):
    A, B = _f32(A), _f32(B)
    Cc = None if C_ is None else _f32(C_)
    Y = np.zeros((M, N), dtype=np.float32)
    load().oracle_gemm_f32(C.c_int(M), C.c_int(N), C.c_int(K), C.c_int(transA), C.c_int(transB), C.c_float(alpha),
                           C.c_float(beta), _ptr(A), _ptr(B), _ptr(Cc), C.c_int(bias_mode), C.c_int(act),
                           C.c_float(act_alpha), _ptr(Y))
    return Y


def unary(x, act, alpha=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    load().oracle_unary(_ptr(y), _ptr(x), C.c_size_t(x.size), C.c_int(act), C.c_float(alpha))
    return y


def unary_chain(x, ops):
    """ops: [(code, alpha, beta)], applied in order (the codes of include/sofie_hip.h)."""
    x = _f32(x)
    y = np.empty_like(x)
    n = len(ops)
    op = (C.c_int * max(n, 1))(*[int(o[0]) for o in ops])
    al = (C.c_float * max(n, 1))(*[float(o[1]) for o in ops])
    be = (C.c_float * max(n, 1))(*[float(o[2]) for o in ops])
    load().oracle_unary_chain(_ptr(y), _ptr(x), C.c_size_t(x.size), C.c_int(n), op, al, be)
    return y


def add_broadcast(A, B):
    A, B = _f32(A), _f32(B)
    yshape = np.broadcast_shapes(A.shape, B.shape)
    rank = len(yshape)
    ash = (1,) * (rank - A.ndim) + A.shape
    bsh = (1,) * (rank - B.ndim) + B.shape
    Y = np.empty(yshape, dtype=np.float32)
    arr = lambda s: (C.c_int64 * 6)(*(list(s) + [1] * (6 - len(s))))
    load().oracle_add_broadcast(C.c_int(rank), arr(yshape), arr(ash), arr(bsh), _ptr(A), _ptr(B), _ptr(Y))
    return Y


def binary_broadcast(A, B, op, param=0.0):
    """op: the SOFIE_BINARY_* code of include/sofie_hip.h."""
    A, B = _f32(A), _f32(B)
    yshape = np.broadcast_shapes(A.shape, B.shape)
    rank = len(yshape)
    ash = (1,) * (rank - A.ndim) + A.shape
    bsh = (1,) * (rank - B.ndim) + B.shape
    Y = np.empty(yshape, dtype=np.float32)
    arr = lambda s: (C.c_int64 * 6)(*(list(s) + [1] * (6 - len(s))))
    load().oracle_binary_broadcast(C.c_int(rank), arr(yshape), arr(ash), arr(bsh), _ptr(A), _ptr(B), _ptr(Y), C.c_int(op), C.c_float(param))
    return Y


def conv_out_hw(H, W, kh, kw, pads, strides, dils):
    OH = (H + pads[0] + pads[2] - (dils[0] * (kh - 1) + 1)) // strides[0] + 1
    OW = (W + pads[1] + pads[3] - (dils[1] * (kw - 1) + 1)) // strides[1] + 1
    return OH, OW


def conv_f32(X, W, bias=None, *, pads=(0, 0, 0, 0), strides=(1, 1), dils=(1, 1), group=1, act=0, act_alpha=0.0):
    """X [N,C,H,W], W [Cout,C/group,kh,kw], pads (h0,w0,h1,w1)."""
    X, W = _f32(X), _f32(W)
    b = None if bias is None else _f32(bias)
    N, Cc, H, Wd = X.shape
    Cout, _, kh, kw = W.shape
    OH, OW = conv_out_hw(H, Wd, kh, kw, pads, strides, dils)
    Y = np.zeros((N, Cout, OH, OW), dtype=np.float32)
    rc = load().oracle_conv_f32(N, Cc, H, Wd, Cout, kh, kw, pads[0], pads[1], pads[2], pads[3], strides[0], strides[1],
                                dils[0], dils[1], group, _ptr(X), _ptr(W), _ptr(b), act, C.c_float(act_alpha), _ptr(Y))
    if rc:
        raise MemoryError("oracle_conv_f32")
    return Y


def conv3d_f32(X, W, bias=None, *, pads=(0, 0, 0, 0, 0, 0), strides=(1, 1, 1), dils=(1, 1, 1), group=1, act=0, act_alpha=0.0):
    """X [N,C,D,H,W], W [Cout,C/group,kd,kh,kw], pads (d0,h0,w0,d1,h1,w1) as the ONNX attribute orders them."""
    X, W = _f32(X), _f32(W)
    b = None if bias is None else _f32(bias)
    N, Cc, D, H, Wd = X.shape
    Cout, _, kd, kh, kw = W.shape
    out = [(X.shape[2 + a] + pads[a] + pads[a + 3] - (dils[a] * (W.shape[2 + a] - 1) + 1)) // strides[a] + 1 for a in range(3)]
    Y = np.zeros((N, Cout, out[0], out[1], out[2]), dtype=np.float32)
    i3 = C.c_int * 3
    rc = load().oracle_conv3d_f32(N, Cc, D, H, Wd, Cout, kd, kh, kw, (C.c_int * 6)(*pads), i3(*strides), i3(*dils), group, _ptr(X), _ptr(W),
                                  _ptr(b), act, C.c_float(act_alpha), _ptr(Y))
    if rc:
        raise MemoryError("oracle_conv3d_f32")
    return Y


def im2col(x, kh, kw, pads, strides, dils):
    """x [C,H,W] -> [C*kh*kw, OH*OW]; pads (h0,w0,h1,w1)."""
    x = _f32(x)
    Cc, H, W = x.shape
    OH, OW = conv_out_hw(H, W, kh, kw, pads, strides, dils)
    col = np.empty((Cc * kh * kw, OH * OW), dtype=np.float32)
    load().oracle_im2col(_ptr(x), Cc, H, W, kh, kw, pads[0], pads[2], pads[1], pads[3], strides[0], strides[1], dils[0],
                         dils[1], _ptr(col))
    return col


def global_avg_pool(X):
    X = _f32(X)
    N, Cc = X.shape[:2]
    HW = int(np.prod(X.shape[2:]))
    Y = np.empty((N, Cc) + (1,) * (X.ndim - 2), dtype=np.float32)
    load().oracle_global_avg_pool(_ptr(Y), _ptr(X), N * Cc, HW)
    return Y


def pool_axes(in_shape, kernel_shape, pads=None, strides=None, dilations=None, auto_pad="NOTSET", ceil_mode=0):
    """Per spatial axis (in, out, window, stride, pad_begin, pad_end): the attribute resolution and output extent of
    core/inc/SOFIE/operators/ROperator_Pool.hxx:107-171 (window = dilated extent, SAME_* padding, ceil_mode limit)."""
    nd = len(in_shape)
    axes = []
    for d in range(nd):
        n_in = int(in_shape[d])
        k = int(kernel_shape[d]) if kernel_shape else n_in
        dil = int(dilations[d]) if dilations else 1
        stride = int(strides[d]) if strides else 1
        window = k + (dil - 1) * (k - 1)
        pb = pe = 0
        if auto_pad == "NOTSET":
            if pads:
                pb, pe = int(pads[d]), int(pads[d + nd])
        elif auto_pad in ("SAME_UPPER", "SAME_LOWER"):
            out_same = (n_in + stride - 1) // stride
            total = max(0, (out_same - 1) * stride + window - n_in)
            pb, pe = (total // 2, total - total // 2) if auto_pad == "SAME_UPPER" else (total - total // 2, total // 2)
        elif auto_pad != "VALID":
            raise ValueError("invalid auto_pad " + auto_pad)
        n = n_in + pb + pe - window
        out = min((n + stride - 1) // stride, (n_in - 1 + pb) // stride) + 1 if ceil_mode else n // stride + 1
        axes.append((n_in, out, window, stride, pb, pe))
    return axes


def pool(X, mode, kernel_shape, pads=None, strides=None, dilations=None, auto_pad="NOTSET", ceil_mode=0, count_include_pad=0):
    """MaxPool (mode "max") / AveragePool (mode "average") of an [N, C, W], [N, C, H, W] or [N, C, D, H, W] tensor."""
    X = _f32(X)
    axes = pool_axes(X.shape[2:], kernel_shape, pads, strides, dilations, auto_pad, ceil_mode)
    if len(axes) == 3:
        planes = X.shape[0] * X.shape[1]
        Y = np.empty(X.shape[:2] + tuple(a[1] for a in axes), dtype=np.float32)
        i3 = lambda col: (C.c_int * 3)(*[a[col] for a in axes])
        lib = load()
        lib.oracle_pool3d.restype = C.c_long
        per_plane = lib.oracle_pool3d(_ptr(Y), _ptr(X), planes, i3(0), i3(2), i3(4), i3(5), i3(3), 1 if mode == "max" else 0, int(ceil_mode),
                                      int(count_include_pad))
        if planes and per_plane != axes[0][1] * axes[1][1] * axes[2][1]:
            raise AssertionError("pool: the loops wrote %d outputs per plane, the shape says %s" % (per_plane, [a[1] for a in axes]))
        return Y
    if len(axes) == 1:
        axes = [(1, 1, 1, 1, 0, 0)] + axes
    (H, OH, kh, sh, ph0, ph1), (W, OW, kw, sw, pw0, pw1) = axes
    planes = X.shape[0] * X.shape[1]
    Y = np.empty(X.shape[:2] + ((OH, OW) if X.ndim == 4 else (OW,)), dtype=np.float32)
    lib = load()
    lib.oracle_pool2d.restype = C.c_long
    per_plane = lib.oracle_pool2d(_ptr(Y), _ptr(X), planes, H, W, kh, kw, ph0, pw0, ph1, pw1, sh, sw, 1 if mode == "max" else 0,
                                  int(ceil_mode), int(count_include_pad))
    # the loops' own count of window positions must be the inferred output shape
    if planes and per_plane != OH * OW:
        raise AssertionError("pool: the loops wrote %d outputs per plane, the shape says %d" % (per_plane, OH * OW))
    return Y


def softmax(X, axis=-1, log=False):
    X = _f32(X)
    axis = axis + X.ndim if axis < 0 else axis
    outer, A, inner = int(np.prod(X.shape[:axis], dtype=np.int64)), X.shape[axis], int(np.prod(X.shape[axis + 1:], dtype=np.int64))
    Y = np.empty_like(X)
    load().oracle_softmax(_ptr(Y), _ptr(X), C.c_long(outer), C.c_int(A), C.c_long(inner), C.c_int(1 if log else 0))
    return Y


def reduce_block(shape, axes):
    """(outer, A, inner) of a reduction over adjacent axes of `shape` (dimensions of 1 may lie between them); None if the axes are not adjacent."""
    rank = len(shape)
    ax = sorted(a + rank if a < 0 else a for a in axes) if axes else list(range(rank))
    if any(shape[i] != 1 for i in range(ax[0], ax[-1] + 1) if i not in ax):
        return None
    return (int(np.prod(shape[:ax[0]], dtype=np.int64)), int(np.prod(shape[ax[0]:ax[-1] + 1], dtype=np.int64)),
            int(np.prod(shape[ax[-1] + 1:], dtype=np.int64)))


def reduce(X, op, axes=None, keepdims=1):
    """op: the SOFIE_REDUCE_* code; axes must be adjacent."""
    X = _f32(X)
    outer, A, inner = reduce_block(X.shape, axes)
    Y = np.empty(outer * inner, dtype=np.float32)
    load().oracle_reduce(_ptr(Y), _ptr(X), C.c_long(outer), C.c_int(A), C.c_long(inner), C.c_int(op))
    rank = X.ndim
    ax = sorted(a + rank if a < 0 else a for a in axes) if axes else list(range(rank))
    shape = [1 if i in ax else d for i, d in enumerate(X.shape)] if keepdims else [d for i, d in enumerate(X.shape) if i not in ax]
    return Y.reshape(shape)


def layernorm(X, scale, bias=None, axis=-1, eps=1e-5, stats=False):
    X, scale = _f32(X), _f32(scale)
    axis = axis + X.ndim if axis < 0 else axis
    rows, L = int(np.prod(X.shape[:axis], dtype=np.int64)), int(np.prod(X.shape[axis:], dtype=np.int64))
    b = None if bias is None else _f32(bias)
    assert scale.size == L and (b is None or b.size == L)
    Y = np.empty_like(X)
    mean, inv = np.empty(rows, np.float32), np.empty(rows, np.float32)
    load().oracle_layernorm(_ptr(Y), _ptr(X), _ptr(scale), _ptr(b), C.c_long(rows), C.c_int(L), C.c_float(eps), _ptr(mean), _ptr(inv))
    return (Y, mean, inv) if stats else Y


def batchnorm(X, scale, bias, mean, var, eps=1e-5, relu=0):
    X = _f32(X)
    Cc = X.shape[1]
    scale, bias, mean, var = _f32(scale), _f32(bias), _f32(mean), _f32(var)
    fused = np.empty(Cc, dtype=np.float32)
    load().oracle_batchnorm_fused_scale(_ptr(fused), _ptr(scale), _ptr(var), Cc, C.c_float(eps))
    Y = np.empty_like(X)
    load().oracle_batchnorm(_ptr(Y), _ptr(X), _ptr(fused), _ptr(mean), _ptr(bias), X.shape[0], Cc, int(np.prod(X.shape[2:])), relu)
    return Y, fused


def global_avg_pool_i8(X, scale):
    X = np.ascontiguousarray(X, dtype=np.int8)
    N, Cc = X.shape[:2]
    HW = int(np.prod(X.shape[2:]))
    Y = np.empty((N, Cc), dtype=np.float32)
    load().oracle_global_avg_pool_i8(_ptr(Y), _ptr(X), N * Cc, HW, C.c_float(scale))
    return Y


def organize_memory(begin, end, size, lib=None, fn="oracle_organize_memory"):
    n = len(begin)
    b = (C.c_int * n)(*begin)
    e = (C.c_int * n)(*end)
    s = (C.c_size_t * n)(*size)
    off = (C.c_size_t * n)()
    tot, tfree, lfree = C.c_size_t(), C.c_size_t(), C.c_size_t()
    lib = lib or load()
    rc = getattr(lib, fn)(n, b, e, s, off, C.byref(tot), C.byref(tfree), C.byref(lfree))
    if rc:
        raise ValueError("organize_memory failed with %d" % rc)
    return {"total_bytes": tot.value, "offsets": list(off), "total_free_bytes": tfree.value,
            "largest_free_block": lfree.value}


def plan_memory_greedy(ops, sizes, model_outputs=()):
    """The reference's CPU-path pool planner.  ops: one (outputs, inputs) pair of tensor-id lists per operator, in execution
    order (inputs that are model inputs or weights: any id < 0); sizes[t]: bytes of tensor t; model_outputs: ids never released.
    A tensor is released after the last operator that reads it (core/src/RModel.cxx:220-249); one that nothing reads has its
    producer as last use (:773-782) but keeps its chunk, because only an operator's inputs are ever released (:606-613).  Returns {"offsets": [...], "pool_bytes": n}."""
    n_t = len(sizes)
    last = [-2] * n_t
    for i, (outs, ins) in enumerate(ops):
        for t in ins:
            if t >= 0:
                last[t] = i
    for i, (outs, ins) in enumerate(ops):
        for t in outs:
            if last[t] == -2:
                last[t] = i
    for t in model_outputs:
        last[t] = -1
    out_ptr, out_ids, in_ptr, in_ids = [0], [], [0], []
    for outs, ins in ops:
        out_ids += list(outs)
        in_ids += list(ins)
        out_ptr.append(len(out_ids))
        in_ptr.append(len(in_ids))
    arr = lambda v: (C.c_int * max(1, len(v)))(*v)
    off = (C.c_size_t * n_t)()
    pool = C.c_size_t()
    rc = load().oracle_plan_memory_greedy(len(ops), arr(out_ptr), arr(out_ids), arr(in_ptr), arr(in_ids), n_t,
                                          (C.c_size_t * n_t)(*sizes), arr(last), off, C.byref(pool))
    if rc:
        raise MemoryError("oracle_plan_memory_greedy")
    return {"offsets": list(off), "pool_bytes": pool.value, "last_use": last}


def quantize_linear(x, scale):
    x = _f32(x)
    q = np.empty(x.shape, dtype=np.int8)
    load().oracle_quantize_linear(_ptr(q), _ptr(x), C.c_size_t(x.size), C.c_float(scale))
    return q


def dequantize_linear(q, scale):
    q = np.ascontiguousarray(q)
    y = np.empty(q.shape, dtype=np.float32)
    if q.dtype == np.int8:
        load().oracle_dequantize_linear_i8(_ptr(y), _ptr(q), C.c_size_t(q.size), C.c_float(scale))
    elif q.dtype == np.int32:
        load().oracle_dequantize_linear_i32(_ptr(y), _ptr(q), C.c_size_t(q.size), C.c_float(scale))
    else:
        raise TypeError(q.dtype)
    return y


_OUT_DTYPE = {0: np.int32, 1: np.float32, 2: np.int8, 3: np.int8}


def matmul_integer(A, B, *, M, N, K, transA=0, transB=0, omp=False):
    A = np.ascontiguousarray(A, dtype=np.int8)
    B = np.ascontiguousarray(B, dtype=np.int8)
    acc = np.empty((M, N), dtype=np.int32)
    load(omp).oracle_matmul_integer(M, N, K, transA, transB, _ptr(A), _ptr(B), _ptr(acc))
    return acc


def gemm_i8_epilogue(acc, *, bias=None, scale=None, scale_scalar=1.0, q_scale=1.0, relu_acc=0, relu_out=0, out=0):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    M, N = acc.shape
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    s = None if scale is None else _f32(scale)
    Y = np.empty((M, N), dtype=_OUT_DTYPE[out])
    load().oracle_gemm_i8_epilogue(M, N, _ptr(acc), _ptr(b), _ptr(s), C.c_float(scale_scalar), C.c_float(q_scale),
                                   relu_acc, relu_out, out, _ptr(Y))
    return Y


def gemm_i8(A, B, *, M, N, K, transA=0, transB=0, omp=False, **epi):
    return gemm_i8_epilogue(matmul_integer(A, B, M=M, N=N, K=K, transA=transA, transB=transB, omp=omp), **epi)


def conv_i8(X, W, bias=None, scale=None, *, pads=(0, 0, 0, 0), strides=(1, 1), dils=(1, 1), group=1, relu=0, out=2,
            omp=False):
    X = np.ascontiguousarray(X, dtype=np.int8)
    W = np.ascontiguousarray(W, dtype=np.int8)
    b = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    s = None if scale is None else _f32(scale)
    N, Cc, H, Wd = X.shape
    Cout, _, kh, kw = W.shape
    OH, OW = conv_out_hw(H, Wd, kh, kw, pads, strides, dils)
    Y = np.empty((N, Cout, OH, OW), dtype=_OUT_DTYPE[out])
    load(omp).oracle_conv_i8(N, Cc, H, Wd, Cout, kh, kw, pads[0], pads[1], pads[2], pads[3], strides[0], strides[1],
                             dils[0], dils[1], group, _ptr(X), _ptr(W), _ptr(b), _ptr(s), relu, out, _ptr(Y))
    return Y


def e4m3_to_f32(codes):
    lib = load()
    codes = np.asarray(codes, dtype=np.uint8)
    lut = np.array([lib.oracle_e4m3_to_f32(i) for i in range(256)], dtype=np.float32)
    return lut[codes]


def quantize_fp8(x, scale):
    x = _f32(x)
    q = np.empty(x.shape, dtype=np.uint8)
    load().oracle_quantize_fp8(_ptr(q), _ptr(x), C.c_size_t(x.size), C.c_float(scale))
    return q


def f32_to_bf16_bits(x):
    lib = load()
    x = _f32(x)
    return np.array([lib.oracle_f32_to_bf16(float(v)) for v in x.ravel()], dtype=np.uint16).reshape(x.shape)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def gemm_fp8(A, B, *, M, N, K, transB=0, bias=None, scale=1.0, act=0, out=1, want_abs_sum=False, omp=False):
    A = np.ascontiguousarray(A, dtype=np.uint8)
    B = np.ascontiguousarray(B, dtype=np.uint8)
    b = None if bias is None else _f32(bias)
    Y = np.empty((M, N), dtype=np.float32 if out == 1 else np.uint16)
    sa = np.empty((M, N), dtype=np.float32) if want_abs_sum else None
    load(omp).oracle_gemm_fp8(M, N, K, transB, _ptr(A), _ptr(B), _ptr(b), C.c_float(scale), act, out, _ptr(Y), _ptr(sa))
    return (Y, sa) if want_abs_sum else Y


def fp8_gemm_bound(A, Bt, bias, scale, act, bf16, omp=True):
    """The per-element bound that include/sofie_hip.h states for sofie_hip_gemm_fp8, evaluated for A [M,K] x Bt [N,K]^T:
    returns (y0, bound) with y0 the fp32 result of exact accumulation."""
    M, K = A.shape
    N = Bt.shape[0]
    scale = np.float32(scale)
    y0, S = gemm_fp8(A, Bt, M=M, N=N, K=K, transB=1, bias=bias, scale=scale, act=act, out=1, want_abs_sum=True, omp=omp)
    v0 = y0 if act == 0 else gemm_fp8(A, Bt, M=M, N=N, K=K, transB=1, bias=bias, scale=scale, act=0, out=1, omp=omp)
    y0 = y0.astype(np.float64)
    v0 = np.abs(v0.astype(np.float64))
    b = np.zeros(N) if bias is None else np.abs(np.asarray(bias, dtype=np.float64))
    lip = 1.13 if act in (4, 5) else 1.0     # SOFIE_ACT_GELU, SOFIE_ACT_GELU_TANH
    bound = lip * (2.0 ** -14 * S.astype(np.float64) * float(scale) + 2.0 ** -22 * (v0 + b[None, :]))
    if act == 4:
        bound = bound + (8e-5 if bf16 else 1e-6) * v0
    bound = bound + 2.0 ** -21 * np.abs(y0)
    if bf16:
        # half an ulp of bf16 (8 significant bits) at the largest magnitude the result may have
        top = np.maximum(np.abs(y0) + bound, 2.0 ** -126)
        bound = bound + np.ldexp(1.0, np.floor(np.log2(top)).astype(np.int64) - 8)
    return y0, bound


def fp8_gemm_bound_excess(got, A, Bt, bias, scale, act, bf16, omp=True):
    """max over the elements of |got - y0| - bound: positive where a result leaves the stated bound."""
    y0, bound = fp8_gemm_bound(A, Bt, bias, scale, act, bf16, omp=omp)
    return float((np.abs(np.asarray(got, dtype=np.float64) - y0) - bound).max())

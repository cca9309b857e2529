"""Runs the small ONNX graphs of the golden fixtures operator by operator, on the CPU oracle or through
the HIP C-ABI.  The operator attribute conventions are the reference's (file:line cited at each)."""
import ctypes as C
import json
import os

import numpy as np

from tests import onnx_lite

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ACT = {"Relu": 1, "LeakyRelu": 2, "Sigmoid": 3, "Gelu": 4, "Tanh": 6}


def load_fixture(model):
    fx = json.load(open(os.path.join(GOLDEN, "fixtures.json")))[model]
    g = onnx_lite.load(os.path.join(GOLDEN, "models", model + ".onnx"))
    inputs = []
    for (name, shape), spec in zip(g["inputs"], fx["inputs"]):
        n = int(np.prod(shape))
        if spec["kind"] == "iota":
            a = np.arange(n, dtype=np.float32)
        elif spec["kind"] == "ones":
            a = np.ones(n, dtype=np.float32)
        else:
            a = np.array(spec["values"], dtype=np.float32)
        inputs.append(a.reshape(shape))
    return g, inputs, np.array(fx["expected"], dtype=np.float32)


def conv_geometry(attrs, xshape, wshape):
    """pads / strides / dilations / group as ROperator_Conv::DoShapeInference resolves them
    (core/inc/SOFIE/operators/ROperator_Conv.hxx:123-262): no `pads` attribute with auto_pad NOTSET means
    pads of 1 (:172-175); SAME_UPPER/LOWER split (:176-197).  Returns 2-D geometry (1-D gets H=1)."""
    dim = len(xshape) - 2
    k = list(attrs.get("kernel_shape", wshape[2:]))
    strides = list(attrs.get("strides", [1] * dim))
    dils = list(attrs.get("dilations", [1] * dim))
    group = attrs.get("group", 1)
    auto = attrs.get("auto_pad", "NOTSET")
    spatial = list(xshape[2:])
    if auto == "NOTSET":
        pads = list(attrs.get("pads", [1] * (2 * dim)))
    elif auto in ("SAME_UPPER", "SAME_LOWER"):
        pads = [0] * (2 * dim)
        for d in range(dim):
            ek = k[d] + (dils[d] - 1) * (k[d] - 1)
            out = (spatial[d] + strides[d] - 1) // strides[d]
            total = max(0, (out - 1) * strides[d] + ek - spatial[d])
            lo, hi = (total // 2, total - total // 2) if auto == "SAME_UPPER" else (total - total // 2, total // 2)
            pads[d], pads[d + dim] = lo, hi
    elif auto == "VALID":
        pads = [0] * (2 * dim)
    else:
        raise ValueError(auto)
    if dim == 3:  # the pads stay in the attribute's order {d0, h0, w0, d1, h1, w1}
        return dict(k=tuple(k), pads=tuple(pads), strides=tuple(strides), dils=tuple(dils), group=group)
    if dim == 1:  # H = 1
        return dict(k=(1, k[0]), pads=(0, pads[0], 0, pads[1]), strides=(1, strides[0]), dils=(1, dils[0]), group=group)
    return dict(k=(k[0], k[1]), pads=(pads[0], pads[1], pads[2], pads[3]), strides=tuple(strides), dils=tuple(dils), group=group)


def fuse(nodes):
    """The parse-time fusions of the reference that matter here: Gemm followed by Relu on its only
    consumer becomes one operator (parsers/src/RModelParser_ONNX.cxx:1208-1212)."""
    out, i = [], 0
    while i < len(nodes):
        n = dict(nodes[i])
        if n["op"] == "Gemm" and i + 1 < len(nodes) and nodes[i + 1]["op"] == "Relu" and nodes[i + 1]["inputs"] == n["outputs"]:
            n["fused_act"] = 1
            n["outputs"] = nodes[i + 1]["outputs"]
            i += 1
        out.append(n)
        i += 1
    return out


class OracleBackend:
    def __init__(self):
        from oracle import binding
        self.ob = binding

    def gemm(self, A, B, Cb, transA, transB, alpha, beta, act):
        M, K = (A.shape[1], A.shape[0]) if transA else A.shape
        N = B.shape[0] if transB else B.shape[1]
        mode = 0 if Cb is None else (4 if Cb.shape == (M, N) else 1 if Cb.size == N else 2 if Cb.size == M else 3)
        return self.ob.gemm_f32(A, B, Cb, M=M, N=N, K=K, transA=transA, transB=transB, alpha=alpha, beta=beta, bias_mode=mode, act=act)

    def unary(self, x, act, alpha):
        return self.ob.unary(x, act, alpha)

    def chain(self, x, ops):
        return self.ob.unary_chain(x, ops)

    def conv(self, X, W, b, geo):
        if X.ndim == 5:
            return self.ob.conv3d_f32(X, W, b, pads=geo["pads"], strides=geo["strides"], dils=geo["dils"], group=geo["group"])
        return self.ob.conv_f32(X, W, b, pads=geo["pads"], strides=geo["strides"], dils=geo["dils"], group=geo["group"])

    def gap(self, X):
        return self.ob.global_avg_pool(X)

    def pool(self, X, mode, a):
        return self.ob.pool(X, mode, a.get("kernel_shape"), a.get("pads"), a.get("strides"), a.get("dilations"), a.get("auto_pad", "NOTSET"),
                            a.get("ceil_mode", 0), a.get("count_include_pad", 0))

    def softmax(self, X, axis, log):
        return self.ob.softmax(X, axis, log)

    def layernorm(self, X, scale, bias, axis, eps):
        return self.ob.layernorm(X, scale, bias, axis, eps)

    def reduce(self, X, op, axes, keepdims):
        return self.ob.reduce(X, op, axes, keepdims)

    # pure data movement: numpy is the definition
    def transpose(self, X, perm):
        return np.ascontiguousarray(np.transpose(X, perm))

    def view(self, X, v):
        """`v`, a numpy view of X (a slice, a broadcast), as a dense tensor"""
        return np.ascontiguousarray(v)

    def take(self, X, indices, axis):
        return np.ascontiguousarray(np.take(X, indices, axis=axis))

    def concat(self, xs, axis):
        return np.ascontiguousarray(np.concatenate(xs, axis=axis))

    def add(self, A, B):
        return self.ob.add_broadcast(A, B)

    def binary(self, A, B, op, param=0.0):
        return self.ob.binary_broadcast(A, B, op, param)


class HipBackend:
    """Every operator goes through the C-ABI on device buffers."""

    def __init__(self, rt):
        from sofie_amd import runtime as R
        from tests import util
        self.rt, self.R, self.u = rt, R, util

    def gemm(self, A, B, Cb, transA, transB, alpha, beta, act):
        R, u = self.R, self.u
        M, K = (A.shape[1], A.shape[0]) if transA else A.shape
        N = B.shape[0] if transB else B.shape[1]
        mode = 0 if Cb is None else (4 if Cb.shape == (M, N) else 1 if Cb.size == N else 2 if Cb.size == M else 3)
        dA, dB = u.to_dev(A), u.to_dev(B)
        dC = None if Cb is None else u.to_dev(Cb)
        dY = u.dev_empty((M, N), np.float32)
        d = R.GemmF32Desc()
        d.M, d.N, d.K, d.transA, d.transB, d.alpha, d.beta = M, N, K, transA, transB, alpha, beta
        d.A, d.B, d.C, d.Y = u.ptr(dA), u.ptr(dB), u.ptr(dC), u.ptr(dY)
        d.bias_mode, d.act, d.batch = mode, act, 1
        import torch
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_gemm_f32", C.byref(d))
        self.rt.sync()
        return u.to_host(dY)

    def unary(self, x, act, alpha):
        u = self.u
        dx = u.to_dev(np.ascontiguousarray(x, dtype=np.float32))
        dy = u.dev_empty(x.shape, np.float32)
        import torch
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_unary_f32", u.ptr(dy), u.ptr(dx), C.c_size_t(x.size), act, C.c_float(alpha))
        self.rt.sync()
        return u.to_host(dy)

    def chain(self, x, ops):
        from sofie_amd.runtime import PostOps
        u = self.u
        dx = u.to_dev(np.ascontiguousarray(x, dtype=np.float32))
        dy = u.dev_empty(x.shape, np.float32)
        import torch
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_unary_chain_f32", u.ptr(dy), u.ptr(dx), C.c_size_t(x.size), C.byref(PostOps.of(ops)))
        self.rt.sync()
        return u.to_host(dy)

    def conv3d(self, X, W, b, geo):
        R, u = self.R, self.u
        N, Cc, D, H, Wd = X.shape
        Cout, _, kd, kh, kw = W.shape
        out = [(X.shape[2 + a] + geo["pads"][a] + geo["pads"][a + 3] - (geo["dils"][a] * (W.shape[2 + a] - 1) + 1)) // geo["strides"][a] + 1 for a in range(3)]
        d = R.Conv3dDesc()
        (d.N, d.C, d.D, d.H, d.W, d.Cout, d.kd, d.kh, d.kw) = (N, Cc, D, H, Wd, Cout, kd, kh, kw)
        d.pad, d.stride, d.dil = (C.c_int32 * 6)(*geo["pads"]), (C.c_int32 * 3)(*geo["strides"]), (C.c_int32 * 3)(*geo["dils"])
        d.group, d.OD, d.OH, d.OW = geo["group"], out[0], out[1], out[2]
        dX, dW = u.to_dev(X), u.to_dev(W)
        db = None if b is None else u.to_dev(b)
        dY = u.dev_empty((N, Cout, out[0], out[1], out[2]), np.float32)
        import torch
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_conv3d_f32", C.byref(d), u.ptr(dX), u.ptr(dW), u.ptr(db), 0, C.c_float(0), u.ptr(dY), None, None)
        self.rt.sync()
        return u.to_host(dY)

    def conv(self, X, W, b, geo):
        if X.ndim == 5:
            return self.conv3d(X, W, b, geo)
        from oracle.binding import conv_out_hw
        R, u = self.R, self.u
        N, Cc, H, Wd = X.shape
        Cout, _, kh, kw = W.shape
        OH, OW = conv_out_hw(H, Wd, kh, kw, geo["pads"], geo["strides"], geo["dils"])
        d = R.ConvDesc()
        (d.N, d.C, d.H, d.W, d.Cout, d.kh, d.kw) = (N, Cc, H, Wd, Cout, kh, kw)
        (d.pad_h0, d.pad_w0, d.pad_h1, d.pad_w1) = geo["pads"]
        (d.stride_h, d.stride_w), (d.dil_h, d.dil_w) = geo["strides"], geo["dils"]
        d.group, d.OH, d.OW = geo["group"], OH, OW
        dX, dW = u.to_dev(X), u.to_dev(W)
        db = None if b is None else u.to_dev(b)
        dY = u.dev_empty((N, Cout, OH, OW), np.float32)
        import torch
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_conv_f32", C.byref(d), u.ptr(dX), u.ptr(dW), u.ptr(db), 0, C.c_float(0), u.ptr(dY), None, None)
        self.rt.sync()
        return u.to_host(dY)

    def gap(self, X):
        u = self.u
        N, Cc = X.shape[:2]
        HW = int(np.prod(X.shape[2:]))
        dX = u.to_dev(X)
        dY = u.dev_empty((N * Cc,), np.float32)
        import torch
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_global_avg_pool_f32", u.ptr(dY), u.ptr(dX), N * Cc, HW)
        self.rt.sync()
        return u.to_host(dY).reshape((N, Cc) + (1,) * (X.ndim - 2))

    def pool(self, X, mode, a):
        from oracle import binding as ob
        R, u = self.R, self.u
        axes = ob.pool_axes(X.shape[2:], a.get("kernel_shape"), a.get("pads"), a.get("strides"), a.get("dilations"), a.get("auto_pad", "NOTSET"),
                            a.get("ceil_mode", 0))
        return hip_pool(self.rt, X, mode, axes, a.get("ceil_mode", 0), a.get("count_include_pad", 0))

    def reduce(self, X, op, axes, keepdims):
        import torch
        from oracle import binding as ob
        u = self.u
        X = np.ascontiguousarray(X, dtype=np.float32)
        outer, A, inner = ob.reduce_block(X.shape, axes)
        dX, dY = u.to_dev(X), u.dev_empty((outer * inner,), np.float32)
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_reduce_f32", u.ptr(dY), u.ptr(dX), outer, A, inner, op)
        self.rt.sync()
        ax = sorted(a + X.ndim if a < 0 else a for a in axes) if axes else list(range(X.ndim))
        shape = [1 if i in ax else d for i, d in enumerate(X.shape)] if keepdims else [d for i, d in enumerate(X.shape) if i not in ax]
        return u.to_host(dY).reshape(shape)

    def layernorm(self, X, scale, bias, axis, eps, stats=False):
        import torch
        u = self.u
        X = np.ascontiguousarray(X, dtype=np.float32)
        axis = axis + X.ndim if axis < 0 else axis
        rows, L = int(np.prod(X.shape[:axis], dtype=np.int64)), int(np.prod(X.shape[axis:], dtype=np.int64))
        dX, dS = u.to_dev(X), u.to_dev(np.ascontiguousarray(scale, dtype=np.float32))
        dB = None if bias is None else u.to_dev(np.ascontiguousarray(bias, dtype=np.float32))
        dY, dM, dI = u.dev_empty(X.shape, np.float32), u.dev_empty((rows,), np.float32), u.dev_empty((rows,), np.float32)
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_layernorm_f32", u.ptr(dY), u.ptr(dX), u.ptr(dS), u.ptr(dB), rows, L, C.c_float(eps), u.ptr(dM) if stats else None,
                     u.ptr(dI) if stats else None)
        self.rt.sync()
        return (u.to_host(dY), u.to_host(dM), u.to_host(dI)) if stats else u.to_host(dY)

    def transpose(self, X, perm):
        import torch
        u = self.u
        X = np.ascontiguousarray(X, dtype=np.float32)
        shape = (C.c_int64 * 6)(*(list(X.shape) + [1] * (6 - X.ndim)))
        p = (C.c_int32 * 6)(*(list(perm) + list(range(X.ndim, 6))))
        dX = u.to_dev(X)
        dY = u.dev_empty(tuple(X.shape[i] for i in perm), np.float32)
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_transpose_f32", u.ptr(dY), u.ptr(dX), X.ndim, shape, p)
        self.rt.sync()
        return u.to_host(dY)

    def view(self, X, v):
        """The strided read that makes the numpy view `v` of the contiguous X dense: shape, element strides and offset are the view's own."""
        import torch
        u = self.u
        assert X.flags["C_CONTIGUOUS"] and X.dtype == np.float32 and v.dtype == np.float32
        dims = [(d, s // 4) for d, s in zip(v.shape, v.strides) if d != 1] or [(1, 0)]       # axes of one element carry no stride
        i = 0
        while i + 1 < len(dims):        # neighbours that walk the input in one stride fold into one axis, as in the emitted Tile
            if dims[i][1] == dims[i + 1][0] * dims[i + 1][1]:
                dims[i:i + 2] = [(dims[i][0] * dims[i + 1][0], dims[i + 1][1])]
            else:
                i += 1
        assert len(dims) <= 6
        offset = (v.__array_interface__["data"][0] - X.__array_interface__["data"][0]) // 4
        shape = (C.c_int64 * 6)(*([d for d, _ in dims] + [1] * (6 - len(dims))))
        strides = (C.c_int64 * 6)(*([s for _, s in dims] + [0] * (6 - len(dims))))
        dX, dY = u.to_dev(X), u.dev_empty(v.shape, np.float32)
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_strided_gather_f32", u.ptr(dY), u.ptr(dX), len(dims), shape, strides, offset, X.size)
        self.rt.sync()
        return u.to_host(dY)

    def take(self, X, indices, axis):
        """one pitched copy per index, as the emitted Gather makes them"""
        import torch
        u = self.u
        X = np.ascontiguousarray(X, dtype=np.float32)
        idx = np.asarray(indices, dtype=np.int64)
        flat = [int(i) + X.shape[axis] if i < 0 else int(i) for i in idx.ravel()]
        outer, inner = int(np.prod(X.shape[:axis], dtype=np.int64)), int(np.prod(X.shape[axis + 1:], dtype=np.int64))
        dX, dY = u.to_dev(X), u.dev_empty(X.shape[:axis] + idx.shape + X.shape[axis + 1:], np.float32)
        torch.cuda.synchronize()
        for k, i in enumerate(flat):
            self.rt.call("sofie_hip_copy_rows", C.c_void_p(u.ptr(dY).value + k * inner * 4), C.c_size_t(len(flat) * inner * 4),
                         C.c_void_p(u.ptr(dX).value + i * inner * 4), C.c_size_t(X.shape[axis] * inner * 4), C.c_size_t(outer), C.c_size_t(inner * 4))
        self.rt.sync()
        return u.to_host(dY)

    def concat(self, xs, axis):
        import torch
        u = self.u
        xs = [np.ascontiguousarray(x, dtype=np.float32) for x in xs]
        axis = axis + xs[0].ndim if axis < 0 else axis
        outer = int(np.prod(xs[0].shape[:axis], dtype=np.int64))
        inner = int(np.prod(xs[0].shape[axis + 1:], dtype=np.int64))
        total = sum(x.shape[axis] for x in xs)
        ysh = xs[0].shape[:axis] + (total,) + xs[0].shape[axis + 1:]
        dY = u.dev_empty(ysh, np.float32)
        devs = [u.to_dev(x) for x in xs]
        torch.cuda.synchronize()
        off = 0
        for x, dx in zip(xs, devs):
            row = x.shape[axis] * inner * 4
            if row:
                self.rt.call("sofie_hip_copy_rows", C.c_void_p(u.ptr(dY).value + off), C.c_size_t(total * inner * 4), u.ptr(dx), C.c_size_t(row), C.c_size_t(outer),
                             C.c_size_t(row))
            off += row
        self.rt.sync()
        return u.to_host(dY)

    def softmax(self, X, axis, log):
        import torch
        u = self.u
        axis = axis + X.ndim if axis < 0 else axis
        outer, A, inner = int(np.prod(X.shape[:axis], dtype=np.int64)), X.shape[axis], int(np.prod(X.shape[axis + 1:], dtype=np.int64))
        dX = u.to_dev(np.ascontiguousarray(X, dtype=np.float32))
        dY = u.dev_empty(X.shape, np.float32)
        torch.cuda.synchronize()
        self.rt.call("sofie_hip_softmax_f32", u.ptr(dY), u.ptr(dX), outer, A, inner, 1 if log else 0)
        self.rt.sync()
        return u.to_host(dY)

    def add(self, A, B):
        return self.binary(A, B, None)

    def binary(self, A, B, op, param=0.0):
        R, u = self.R, self.u
        A, B = np.ascontiguousarray(A, dtype=np.float32), np.ascontiguousarray(B, dtype=np.float32)
        ysh = np.broadcast_shapes(A.shape, B.shape)
        rank = len(ysh)
        d = R.AddDesc()
        d.rank = rank
        for i, v in enumerate(ysh):
            d.y_shape[i] = v
        for i, v in enumerate((1,) * (rank - A.ndim) + tuple(A.shape)):
            d.a_shape[i] = v
        for i, v in enumerate((1,) * (rank - B.ndim) + tuple(B.shape)):
            d.b_shape[i] = v
        dA, dB = u.to_dev(A), u.to_dev(B)
        dY = u.dev_empty(ysh, np.float32)
        d.A, d.B, d.Y = u.ptr(dA), u.ptr(dB), u.ptr(dY)
        import torch
        torch.cuda.synchronize()
        if op is None:
            self.rt.call("sofie_hip_add_f32", C.byref(d))
        else:
            self.rt.call("sofie_hip_binary_f32", C.byref(d), op, C.c_float(param))
        self.rt.sync()
        return u.to_host(dY)


def hip_pool(rt, X, mode, axes, ceil_mode=0, count_include_pad=0):
    """sofie_hip_pool_f32 on an [N, C, (H,) W] array, sofie_hip_pool3d_f32 on [N, C, D, H, W]; axes = per spatial axis (in, out, window, stride, pad_begin, pad_end)."""
    import torch
    from sofie_amd import runtime as R
    from tests import util as u
    if len(axes) == 3:
        col = lambda c: (C.c_int32 * 3)(*[a[c] for a in axes])
        d = R.Pool3dDesc(planes=X.shape[0] * X.shape[1], in_=col(0), out=col(1), k=col(2), stride=col(3), pad_begin=col(4), pad_end=col(5),
                         mode=R.POOL_MAX if mode == "max" else R.POOL_AVERAGE, count_include_pad=int(count_include_pad),
                         dynamic_divisor=int(bool(ceil_mode) or any(a[4] > 0 or a[5] > 0 for a in axes)))
        dX = u.to_dev(np.ascontiguousarray(X, dtype=np.float32))
        dY = u.dev_empty(X.shape[:2] + tuple(a[1] for a in axes), np.float32)
        torch.cuda.synchronize()
        rt.call("sofie_hip_pool3d_f32", C.byref(d), u.ptr(dY), u.ptr(dX))
        rt.sync()
        return u.to_host(dY)
    if len(axes) == 1:
        axes = [(1, 1, 1, 1, 0, 0)] + list(axes)
    (H, OH, kh, sh, ph0, ph1), (W, OW, kw, sw, pw0, pw1) = axes
    d = R.PoolDesc(planes=X.shape[0] * X.shape[1], H=H, W=W, OH=OH, OW=OW, kh=kh, kw=kw, pad_h0=ph0, pad_w0=pw0, pad_h1=ph1, pad_w1=pw1,
                   stride_h=sh, stride_w=sw, mode=R.POOL_MAX if mode == "max" else R.POOL_AVERAGE, count_include_pad=int(count_include_pad),
                   dynamic_divisor=int(bool(ceil_mode) or any(v > 0 for v in (ph0, ph1, pw0, pw1))))
    ysh = X.shape[:2] + ((OH, OW) if X.ndim == 4 else (OW,))
    dX = u.to_dev(np.ascontiguousarray(X, dtype=np.float32))
    dY = u.dev_empty(ysh, np.float32)
    torch.cuda.synchronize()
    rt.call("sofie_hip_pool_f32", C.byref(d), u.ptr(dY), u.ptr(dX))
    rt.sync()
    return u.to_host(dY)


# SOFIE_REDUCE_* codes of include/sofie_hip.h
REDUCE = {"ReduceSum": 0, "ReduceMean": 1, "ReduceSumSquare": 2, "ReduceProd": 3, "ReduceL2": 4, "ReduceMax": 5, "ReduceMin": 6}

# SOFIE_BINARY_* codes of include/sofie_hip.h
BINARY = {"Sub": 1, "Mul": 2, "Div": 3, "Pow": 4}
NARY = {"Max": 5, "Min": 6, "Sum": 0, "Mean": 0}

# codes of include/sofie_hip.h for the reference's basic unary operators
BASIC_UNARY = {"Reciprocal": 7, "Sqrt": 8, "Neg": 9, "Exp": 10, "Log": 11, "Sin": 12, "Cos": 13, "Abs": 14, "Softplus": 15, "Atan": 16,
               "Floor": 17, "Asinh": 18, "Acosh": 19, "Atanh": 20}


def run(g, inputs, be, all_outputs=False):
    env = dict(g["initializers"])
    for (name, _), a in zip(g["inputs"], inputs):
        env[name] = a
    for n in fuse(g["nodes"]):
        op, a = n["op"], n["attrs"]
        x = [env[i] if i else None for i in n["inputs"]]
        if op == "Gemm":
            y = be.gemm(x[0], x[1], x[2] if len(x) > 2 else None, a.get("transA", 0), a.get("transB", 0), a.get("alpha", 1.0),
                        a.get("beta", 1.0), n.get("fused_act", 0))
        elif op in ("Relu", "Sigmoid", "Tanh"):
            y = be.unary(x[0], ACT[op], 0.0)
        elif op == "LeakyRelu":
            y = be.unary(x[0], 2, a.get("alpha", 0.01))
        elif op == "Gelu":
            y = be.unary(x[0], 5 if a.get("approximate", "none") == "tanh" else 4, 0.0)
        elif op in BASIC_UNARY:
            y = be.unary(x[0], BASIC_UNARY[op], 0.0)
        elif op == "Flatten":
            ax = a.get("axis", 1)
            y = np.ascontiguousarray(x[0]).reshape(int(np.prod(x[0].shape[:ax], dtype=np.int64)), -1)
        elif op == "Reshape":
            shape = [int(v) for v in np.asarray(x[1]).ravel()]
            shape = [x[0].shape[i] if (v == 0 and not a.get("allowzero", 0)) else v for i, v in enumerate(shape)]
            y = np.ascontiguousarray(x[0]).reshape(shape)
        elif op in ("Squeeze", "Unsqueeze"):
            axes = [int(v) for v in np.asarray(x[1]).ravel()] if len(x) > 1 and x[1] is not None else list(a.get("axes", []))
            if op == "Squeeze":
                y = np.squeeze(x[0], axis=tuple(axes) if axes else None)
            else:
                y = np.expand_dims(x[0], axis=tuple(axes))
            y = np.ascontiguousarray(y)
        elif op == "Transpose":
            y = be.transpose(x[0], a.get("perm", list(range(x[0].ndim))[::-1]))
        elif op == "Concat":
            y = be.concat(x, a.get("axis", 0))
        elif op == "Slice":
            X = np.ascontiguousarray(x[0], dtype=np.float32)
            par = [[int(v) for v in np.asarray(t).ravel()] if t is not None else None for t in x[1:]] if len(x) > 1 else [a["starts"], a["ends"], a.get("axes")]
            par += [None] * (4 - len(par))
            starts, ends, axes, steps = par[0], par[1], par[2] or list(range(len(par[0]))), par[3] or [1] * len(par[0])
            sl = [slice(None)] * X.ndim
            for s, e, ax, st in zip(starts, ends, axes, steps):       # Python's slices clamp as ONNX's do; an end below -dim means "to the front"
                d = X.shape[ax]
                sl[ax] = slice(max(s, -d) if st > 0 else s, None if (st < 0 and e < -d) else e, st)
            y = be.view(X, X[tuple(sl)])
        elif op == "Split":
            X = np.ascontiguousarray(x[0], dtype=np.float32)
            ax = a.get("axis", 0) % X.ndim
            k = len(n["outputs"])
            if len(x) > 1 and x[1] is not None:
                sizes = [int(v) for v in np.asarray(x[1]).ravel()]
            else:
                per = -(-X.shape[ax] // k)
                sizes = [per] * (k - 1) + [X.shape[ax] - per * (k - 1)]
            start = 0
            for name, sz in zip(n["outputs"], sizes):
                sl = [slice(None)] * X.ndim
                sl[ax] = slice(start, start + sz)
                env[name] = be.view(X, X[tuple(sl)])
                start += sz
            continue
        elif op == "Expand":
            X = np.ascontiguousarray(x[0], dtype=np.float32)
            target = np.broadcast_shapes(X.shape, tuple(int(v) for v in np.asarray(x[1]).ravel()))
            y = be.view(X, np.broadcast_to(X, target))
        elif op == "Tile":
            X = np.ascontiguousarray(x[0], dtype=np.float32)
            reps = [int(v) for v in np.asarray(x[1]).ravel()]
            pairs = np.broadcast_to(X.reshape([v for d in X.shape for v in (1, d)]), [v for r, d in zip(reps, X.shape) for v in (r, d)])
            y = be.view(X, pairs).reshape([r * d for r, d in zip(reps, X.shape)])
            assert np.array_equal(y, np.tile(X, reps)) or not isinstance(be, OracleBackend)
        elif op == "Gather":
            y = be.take(np.ascontiguousarray(x[0], dtype=np.float32), np.asarray(x[1]), a.get("axis", 0) % np.ndim(x[0]))
        elif op == "Selu":
            y = be.chain(x[0], [(22, a.get("alpha", 1.6732631921768188), a.get("gamma", 1.0507010221481323))])
        elif op == "Elu":
            y = be.chain(x[0], [(23, a.get("alpha", 1.0), 0.0)])
        elif op == "Erf":
            y = be.unary(x[0], 24, 0.0)
        elif op == "HardSigmoid":
            y = be.chain(x[0], [(25, a.get("alpha", 0.2), a.get("beta", 0.5))])
        elif op == "HardSwish":
            y = be.unary(x[0], 26, 0.0)
        elif op == "Swish":
            y = be.unary(x[0], 27, 0.0)
        elif op == "Identity":
            y = np.array(x[0], copy=True)
        elif op == "Clip":
            lo = float(np.asarray(x[1]).ravel()[0]) if len(x) > 1 and x[1] is not None else a.get("min", float(np.finfo(np.float32).min))
            hi = float(np.asarray(x[2]).ravel()[0]) if len(x) > 2 and x[2] is not None else a.get("max", float(np.finfo(np.float32).max))
            y = be.chain(x[0], [(21, lo, hi)])
        elif op == "Conv":
            X, W = x[0], x[1]
            b = x[2] if len(x) > 2 else None
            geo = conv_geometry(a, X.shape, W.shape)
            one_d = X.ndim == 3
            if one_d:
                X, W = X[:, :, None, :], W[:, :, None, :]
            y = be.conv(np.ascontiguousarray(X), np.ascontiguousarray(W), b, geo)
            if one_d:
                y = y[:, :, 0, :]
        elif op == "GlobalAveragePool":
            y = be.gap(x[0])
        elif op in REDUCE:
            axes = [int(v) for v in np.asarray(x[1]).ravel()] if len(x) > 1 and x[1] is not None else list(a.get("axes", []))
            y = be.reduce(x[0], REDUCE[op], axes, a.get("keepdims", 1))
        elif op == "LayerNormalization":
            y = be.layernorm(x[0], x[1], x[2] if len(x) > 2 else None, a.get("axis", -1), a.get("epsilon", 1e-5))
        elif op in ("Softmax", "LogSoftmax"):
            y = be.softmax(x[0], a.get("axis", -1), op == "LogSoftmax")
        elif op in ("MaxPool", "AveragePool"):
            y = be.pool(x[0], "max" if op == "MaxPool" else "average", a)
        elif op == "BatchNormalization":
            from oracle import binding as ob
            y, _ = ob.batchnorm(x[0], x[1], x[2], x[3], x[4], eps=a.get("epsilon", 1e-5))
        elif op == "Add":
            y = be.add(x[0], x[1])
        elif op in BINARY:
            y = be.binary(x[0], x[1], BINARY[op])
        elif op in NARY:
            # a left fold of pairwise steps; Mean's last step divides by the number of operands
            y = x[0] if len(x) > 1 else be.binary(x[0], x[0], NARY["Max"])
            for i in range(1, len(x)):
                last = i == len(x) - 1
                y = be.binary(y, x[i], 7 if (op == "Mean" and last) else NARY[op], float(len(x)))
            if op == "Mean" and len(x) == 1:
                y = np.array(x[0], copy=True)
        else:
            raise NotImplementedError(op)
        env[n["outputs"][0]] = y
    if all_outputs:
        return [env[o[0]] for o in g["outputs"]]
    return env[g["outputs"][0][0]]

"""Host-side Session objects that drive the C-ABI the way the emitted C++ Session does: one arena,
weights uploaded (and re-laid out) once at construction, `infer` enqueues the launches on the
context's stream.  Used by the tests and the benchmark; torch only supplies nothing here -- all device
memory is the runtime's arena.
"""
import ctypes as C

import numpy as np

from . import runtime as R


def _align(v, a=256):
    return (v + a - 1) // a * a


class Int8MLPSession:
    """QuantizeLinear -> [int8 Gemm (int32 accumulate) -> Relu -> DequantizeLinear -> QuantizeLinear]* ->
    int8 Gemm -> Relu -> DequantizeLinear, per-tensor symmetric scales.

    The DequantizeLinear/QuantizeLinear pair between two layers is fused into the producing Gemm's store
    (SOFIE_I8OUT_I8_DQQ: the same fp32 multiply, divide and round-half-even, in the same order), so an
    inter-layer activation is written once as int8 and never as fp32.

    weights: list of int8 arrays [K_l, N_l] (the B operand of MatMulInteger); w_scales / in_scales: one
    fp32 scale per layer for the weight and for the layer's quantised input.
    """

    def __init__(self, rt, weights, w_scales, in_scales, batch):
        self.rt = rt
        self.batch = int(batch)
        self.dims = [weights[0].shape[0]] + [w.shape[1] for w in weights]
        self.nlayers = len(weights)
        self.w_scales = [np.float32(s) for s in w_scales]
        self.in_scales = [np.float32(s) for s in in_scales]
        # fp32 product formed once on the host, as the emitted code would hold it as a constant
        self.dq_scales = [np.float32(self.in_scales[l] * self.w_scales[l]) for l in range(self.nlayers)]
        M = self.batch
        off = 0
        self.off_w = []
        for w in weights:
            self.off_w.append(off)
            off = _align(off + w.size)
        stage = max(w.size for w in weights)
        self.off_stage = off
        off = _align(off + stage)
        self.off_x = off
        off = _align(off + 4 * M * self.dims[0])
        self.off_xq = off
        off = _align(off + M * self.dims[0])
        act = max(self.dims[1:-1]) if self.nlayers > 1 else 0
        self.off_act = [off, _align(off + M * act)]
        off = _align(self.off_act[1] + M * act)
        self.off_y = off
        off = _align(off + 4 * M * self.dims[-1])
        rt.call("sofie_hip_arena_create", C.c_size_t(off), C.c_size_t(256))
        self.arena_bytes = off
        p = lambda o: C.c_void_p(rt.lib.sofie_hip_arena_ptr(rt.ctx, C.c_size_t(o)))
        self.p = p
        # weights: upload [K,N], re-lay out once to [N,K] (K contiguous, what the MFMA kernel reads)
        for l, w in enumerate(weights):
            w = np.ascontiguousarray(w, dtype=np.int8)
            K, N = w.shape
            rt.call("sofie_hip_upload", p(self.off_stage), w.ctypes.data_as(C.c_void_p), C.c_size_t(w.size))
            rt.call("sofie_hip_transpose_i8", p(self.off_w[l]), p(self.off_stage), K, N, 0, 0)
            rt.sync()
        self.descs = []
        src = self.off_xq
        for l in range(self.nlayers):
            d = R.GemmI8Desc()
            d.M, d.N, d.K = M, self.dims[l + 1], self.dims[l]
            d.transA, d.transB = 0, 1
            d.A = p(src)
            d.B = p(self.off_w[l])
            d.bias = None
            d.scale = None
            d.scale_scalar = float(self.dq_scales[l])
            d.relu_acc, d.relu_out = 1, 0
            if l + 1 < self.nlayers:
                d.out = R.I8OUT_I8_DQQ
                d.q_scale = float(self.in_scales[l + 1])
                dst = self.off_act[l % 2]
            else:
                d.out = R.I8OUT_F32
                d.q_scale = 1.0
                dst = self.off_y
            d.Y = p(dst)
            src = dst
            self.descs.append(d)

    @property
    def x_ptr(self):
        return self.p(self.off_x)

    @property
    def y_ptr(self):
        return self.p(self.off_y)

    def upload_input(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        assert x.shape == (self.batch, self.dims[0])
        self.rt.call("sofie_hip_upload", self.x_ptr, x.ctypes.data_as(C.c_void_p), C.c_size_t(x.nbytes))

    def infer_nosync(self):
        """Enqueue one inference over the input resident at x_ptr; the result lands at y_ptr."""
        rt = self.rt
        rt.call("sofie_hip_quantize_linear", self.p(self.off_xq), self.x_ptr, C.c_size_t(self.batch * self.dims[0]),
                C.c_float(float(self.in_scales[0])))
        for d in self.descs:
            rt.call("sofie_hip_gemm_i8", C.byref(d))

    def infer(self, x):
        self.upload_input(x)
        self.infer_nosync()
        y = np.empty((self.batch, self.dims[-1]), dtype=np.float32)
        self.rt.call("sofie_hip_download", y.ctypes.data_as(C.c_void_p), self.y_ptr, C.c_size_t(y.nbytes))
        self.rt.sync()
        return y


class Int8CNNSession:
    """QuantizeLinear -> [int8 Conv (int32 accumulate, bias) -> per-channel requantisation -> Relu]* ->
    GlobalAveragePool -> fp32 Gemm: the shape of a CNN whose BatchNorm layers are folded into the
    per-channel scales and biases.  The input is fp32 NCHW (the ONNX layout); the first convolution reads
    its quantised form as NCHW and writes NHWC, every later activation stays NHWC int8, written once.

    convs: list of dicts with W int8 [Cout,Cin,kh,kw], bias int32 [Cout], scale fp32 [Cout]
    (= s_in * s_w[co] / s_out), pads (h0,w0,h1,w1), strides, dils.  fc_w is fp32 [C_last, n_out], fc_b [n_out].
    """

    def __init__(self, rt, batch, in_shape, in_scale, convs, last_scale, fc_w, fc_b, pool_in_conv=True):
        """pool_in_conv: let the last convolution add its planes up in its store (the feature map the average reads is then
        neither written nor read back) whenever the runtime takes that shape; False keeps the two kernels apart."""
        self.rt = rt
        self.batch = N = int(batch)
        Cin, H, W = in_shape
        self.in_shape = (Cin, H, W)
        self.in_scale = np.float32(in_scale)
        self.last_scale = np.float32(last_scale)
        self.conv_descs = []
        shapes = []
        c, h, w = Cin, H, W
        for cv in convs:
            Wt = cv["W"]
            d = R.ConvDesc()
            d.N, d.C, d.H, d.W = N, c, h, w
            d.Cout, d.kh, d.kw = Wt.shape[0], Wt.shape[2], Wt.shape[3]
            d.pad_h0, d.pad_w0, d.pad_h1, d.pad_w1 = cv.get("pads", (0, 0, 0, 0))
            d.stride_h, d.stride_w = cv.get("strides", (1, 1))
            d.dil_h, d.dil_w = cv.get("dils", (1, 1))
            d.group = 1
            d.OH = (h + d.pad_h0 + d.pad_h1 - d.dil_h * (d.kh - 1) - 1) // d.stride_h + 1
            d.OW = (w + d.pad_w0 + d.pad_w1 - d.dil_w * (d.kw - 1) - 1) // d.stride_w + 1
            self.conv_descs.append(d)
            c, h, w = d.Cout, d.OH, d.OW
            shapes.append((c, h, w))
        self.out_shape = shapes[-1]
        self.n_out = fc_w.shape[1]
        lib = rt.lib
        # arena layout
        off = 0

        def take(nbytes):
            nonlocal off
            o = off
            off = _align(off + nbytes)
            return o
        self.off_x = take(4 * N * Cin * H * W)
        self.off_xq = take(N * Cin * H * W)
        act_bytes = max(N * s[0] * s[1] * s[2] for s in shapes)
        self.off_act = [take(act_bytes), take(act_bytes)]
        self.off_wp, self.off_bias, self.off_scale = [], [], []
        for d, cv in zip(self.conv_descs, convs):
            self.off_wp.append(take(lib.sofie_hip_conv_weight_i8_packed_bytes(C.byref(d))))
            self.off_bias.append(take(4 * d.Cout))
            self.off_scale.append(take(4 * d.Cout))
        stage = max(cv["W"].size for cv in convs)
        self.off_stage = take(stage)
        self.off_pool = take(4 * N * self.out_shape[0])
        self.off_sums = take(4 * N * self.out_shape[0])
        self.off_fcw = take(4 * fc_w.size)
        self.off_fcb = take(4 * fc_b.size)
        self.off_y = take(4 * N * self.n_out)
        args0 = R.ConvI8Args()
        args0.w_is_packed = 1
        ws_min = max(lib.sofie_hip_conv_i8_workspace(C.byref(d), C.byref(args0)) for d in self.conv_descs)
        # room for the column matrix of as many images as the runtime will take at once (it caps a chunk itself)
        self.ws_bytes = _align(min(ws_min * N, 200 << 20) if ws_min * N > ws_min else ws_min)
        self.ws_bytes = max(self.ws_bytes, _align(ws_min))
        self.off_ws = take(self.ws_bytes)
        rt.call("sofie_hip_arena_create", C.c_size_t(off), C.c_size_t(256))
        self.arena_bytes = off
        p = lambda o: C.c_void_p(lib.sofie_hip_arena_ptr(rt.ctx, C.c_size_t(o)))
        self.p = p

        def upload(o, a):
            a = np.ascontiguousarray(a)
            rt.call("sofie_hip_upload", p(o), a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes))
            rt.sync()
        self.conv_args = []
        src, src_layout = self.off_xq, R.LAYOUT_NCHW
        for l, (d, cv) in enumerate(zip(self.conv_descs, convs)):
            upload(self.off_stage, cv["W"].astype(np.int8))
            rt.call("sofie_hip_pack_conv_weight_i8", C.byref(d), p(self.off_wp[l]), p(self.off_stage))
            rt.sync()
            upload(self.off_bias[l], cv["bias"].astype(np.int32))
            upload(self.off_scale[l], cv["scale"].astype(np.float32))
            a = R.ConvI8Args()
            a.X, a.W, a.bias, a.scale = p(src), p(self.off_wp[l]), p(self.off_bias[l]), p(self.off_scale[l])
            a.relu, a.out = 1, R.I8OUT_I8
            a.x_layout, a.y_layout, a.w_is_packed = src_layout, R.LAYOUT_NHWC, 1
            dst = self.off_act[l % 2]
            a.Y, a.workspace, a.workspace_bytes = p(dst), p(self.off_ws), self.ws_bytes
            self.conv_args.append(a)
            src, src_layout = dst, R.LAYOUT_NHWC
        self.off_last = src
        # the last convolution may hand the average its plane sums instead of the feature map
        last_d, last_a = self.conv_descs[-1], self.conv_args[-1]
        self.pool_in_conv = bool(pool_in_conv) and (last_d.OH * last_d.OW) % 256 == 0 and \
            lib.sofie_hip_conv_i8_workspace(C.byref(last_d), C.byref(last_a)) == 0
        if self.pool_in_conv:
            last_a.out, last_a.Y = R.I8OUT_I8_PLANE_SUMS, p(self.off_sums)
        upload(self.off_fcw, fc_w.astype(np.float32))
        upload(self.off_fcb, fc_b.astype(np.float32))
        g = R.GemmF32Desc()
        g.M, g.N, g.K = N, self.n_out, self.out_shape[0]
        g.alpha, g.beta = 1.0, 1.0
        g.A, g.B, g.C, g.Y = p(self.off_pool), p(self.off_fcw), p(self.off_fcb), p(self.off_y)
        g.bias_mode, g.act, g.batch = R.BIAS_ROW, R.ACT_NONE, 1
        self.fc = g

    @property
    def x_ptr(self):
        return self.p(self.off_x)

    @property
    def y_ptr(self):
        return self.p(self.off_y)

    def upload_input(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        assert x.shape == (self.batch,) + self.in_shape
        self.rt.call("sofie_hip_upload", self.x_ptr, x.ctypes.data_as(C.c_void_p), C.c_size_t(x.nbytes))

    def infer_nosync(self):
        rt = self.rt
        Cin, H, W = self.in_shape
        rt.call("sofie_hip_quantize_linear", self.p(self.off_xq), self.x_ptr, C.c_size_t(self.batch * Cin * H * W),
                C.c_float(float(self.in_scale)))
        c, h, w = self.out_shape
        if self.pool_in_conv:
            rt.call("sofie_hip_fill_zero", self.p(self.off_sums), C.c_size_t(4 * self.batch * c))
        for d, a in zip(self.conv_descs, self.conv_args):
            rt.call("sofie_hip_conv_i8", C.byref(d), C.byref(a))
        if self.pool_in_conv:
            rt.call("sofie_hip_plane_sums_to_average", self.p(self.off_pool), self.p(self.off_sums), self.batch * c, h * w,
                    C.c_float(float(self.last_scale)))
        else:
            rt.call("sofie_hip_global_avg_pool_i8", self.p(self.off_pool), self.p(self.off_last), self.batch, c, h * w, R.LAYOUT_NHWC,
                    C.c_float(float(self.last_scale)))
        rt.call("sofie_hip_gemm_f32", C.byref(self.fc))

    def infer(self, x):
        self.upload_input(x)
        self.infer_nosync()
        y = np.empty((self.batch, self.n_out), dtype=np.float32)
        self.rt.call("sofie_hip_download", y.ctypes.data_as(C.c_void_p), self.y_ptr, C.c_size_t(y.nbytes))
        self.rt.sync()
        return y

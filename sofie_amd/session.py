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

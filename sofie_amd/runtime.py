"""ctypes view of the C-ABI in include/sofie_hip.h (used by tests/ and bench.py).

There is no fallback: if the library is not built, loading raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))


def lib_path():
    return os.path.join(_HERE, "lib", "libsofie_hip.so")


class SofieHipError(RuntimeError):
    pass


# activation / bias / output codes of include/sofie_hip.h
(ACT_NONE, ACT_RELU, ACT_LEAKYRELU, ACT_SIGMOID, ACT_GELU, ACT_GELU_TANH, ACT_TANH, ACT_RECIPROCAL, ACT_SQRT, ACT_NEG, ACT_EXP, ACT_LOG,
 ACT_SIN, ACT_COS, ACT_ABS, ACT_SOFTPLUS, ACT_ATAN, ACT_FLOOR, ACT_ASINH, ACT_ACOSH, ACT_ATANH, ACT_CLIP, ACT_SELU, ACT_ELU, ACT_ERF, ACT_HARDSIGMOID, ACT_HARDSWISH, ACT_SWISH) = range(28)
MAX_POST_OPS = 4
BIAS_NONE, BIAS_ROW, BIAS_COL, BIAS_SCALAR, BIAS_FULL = range(5)
I8OUT_I32, I8OUT_F32, I8OUT_I8, I8OUT_I8_DQQ, I8OUT_I8_PLANE_SUMS = range(5)
F8OUT_BF16, F8OUT_F32 = range(2)
LAYOUT_NCHW, LAYOUT_NHWC = range(2)


class PostOps(C.Structure):
    _fields_ = [("count", C.c_int32), ("op", C.c_int32 * MAX_POST_OPS), ("alpha", C.c_float * MAX_POST_OPS), ("beta", C.c_float * MAX_POST_OPS)]

    @classmethod
    def of(cls, ops):
        """ops: [(code, alpha, beta)]"""
        p = cls()
        p.count = len(ops)
        for i, (o, a, b) in enumerate(ops[:MAX_POST_OPS]):
            p.op[i], p.alpha[i], p.beta[i] = o, a, b
        return p


class GemmF32Desc(C.Structure):
    _fields_ = [("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("transA", C.c_int32), ("transB", C.c_int32),
                ("lda", C.c_int32), ("ldb", C.c_int32), ("ldy", C.c_int32), ("alpha", C.c_float), ("beta", C.c_float),
                ("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p), ("bias_mode", C.c_int32), ("act", C.c_int32),
                ("act_alpha", C.c_float), ("Y", C.c_void_p), ("batch", C.c_int32), ("strideA", C.c_int64),
                ("strideB", C.c_int64), ("strideC", C.c_int64), ("strideY", C.c_int64), ("post", C.POINTER(PostOps)),
                ("residual", C.c_void_p)]


class GemmI8Desc(C.Structure):
    _fields_ = [("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("transA", C.c_int32), ("transB", C.c_int32),
                ("lda", C.c_int32), ("ldb", C.c_int32), ("ldy", C.c_int32), ("A", C.c_void_p), ("B", C.c_void_p),
                ("bias", C.c_void_p), ("scale", C.c_void_p), ("scale_scalar", C.c_float), ("q_scale", C.c_float),
                ("relu_acc", C.c_int32), ("relu_out", C.c_int32), ("out", C.c_int32), ("Y", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class GemmFp8Desc(C.Structure):
    _fields_ = [("M", C.c_int32), ("N", C.c_int32), ("K", C.c_int32), ("transB", C.c_int32), ("lda", C.c_int32),
                ("ldb", C.c_int32), ("ldy", C.c_int32), ("A", C.c_void_p), ("B", C.c_void_p), ("bias", C.c_void_p),
                ("scale", C.c_float), ("act", C.c_int32), ("out", C.c_int32), ("Y", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class AddDesc(C.Structure):
    _fields_ = [("rank", C.c_int32), ("y_shape", C.c_int64 * 6), ("a_shape", C.c_int64 * 6), ("b_shape", C.c_int64 * 6),
                ("A", C.c_void_p), ("B", C.c_void_p), ("Y", C.c_void_p)]


class ConvDesc(C.Structure):
    _fields_ = [("N", C.c_int32), ("C", C.c_int32), ("H", C.c_int32), ("W", C.c_int32), ("Cout", C.c_int32),
                ("kh", C.c_int32), ("kw", C.c_int32), ("pad_h0", C.c_int32), ("pad_w0", C.c_int32),
                ("pad_h1", C.c_int32), ("pad_w1", C.c_int32), ("stride_h", C.c_int32), ("stride_w", C.c_int32),
                ("dil_h", C.c_int32), ("dil_w", C.c_int32), ("group", C.c_int32), ("OH", C.c_int32), ("OW", C.c_int32)]


class PoolDesc(C.Structure):
    _fields_ = [(name, C.c_int32) for name in ("planes", "H", "W", "OH", "OW", "kh", "kw", "pad_h0", "pad_w0", "pad_h1", "pad_w1",
                                               "stride_h", "stride_w", "mode", "count_include_pad", "dynamic_divisor")]


class Pool3dDesc(C.Structure):
    _fields_ = [("planes", C.c_int32), ("in_", C.c_int32 * 3), ("out", C.c_int32 * 3), ("k", C.c_int32 * 3), ("pad_begin", C.c_int32 * 3),
                ("pad_end", C.c_int32 * 3), ("stride", C.c_int32 * 3), ("mode", C.c_int32), ("count_include_pad", C.c_int32),
                ("dynamic_divisor", C.c_int32)]


POOL_MAX, POOL_AVERAGE = 0, 1
REDUCE_SUM, REDUCE_MEAN, REDUCE_SUM_SQUARE, REDUCE_PROD, REDUCE_L2, REDUCE_MAX, REDUCE_MIN = range(7)
BINARY_ADD, BINARY_SUB, BINARY_MUL, BINARY_DIV, BINARY_POW, BINARY_MAX, BINARY_MIN, BINARY_ADD_DIV = range(8)


class Conv3dDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("N", "C", "D", "H", "W", "Cout", "kd", "kh", "kw")] + \
               [("pad", C.c_int32 * 6), ("stride", C.c_int32 * 3), ("dil", C.c_int32 * 3), ("group", C.c_int32),
                ("OD", C.c_int32), ("OH", C.c_int32), ("OW", C.c_int32)]


class ConvI8Args(C.Structure):
    _fields_ = [("X", C.c_void_p), ("W", C.c_void_p), ("bias", C.c_void_p), ("scale", C.c_void_p),
                ("relu", C.c_int32), ("out", C.c_int32), ("x_layout", C.c_int32), ("y_layout", C.c_int32),
                ("w_is_packed", C.c_int32), ("Y", C.c_void_p), ("workspace", C.c_void_p),
                ("workspace_bytes", C.c_size_t)]


# every symbol include/sofie_hip.h declares: name -> (restype, argtypes)
_P = C.c_void_p
SYMBOLS = {
    "sofie_hip_ctx_create": (C.c_int, [C.POINTER(_P), C.c_int, _P]),
    "sofie_hip_ctx_destroy": (C.c_int, [_P]),
    "sofie_hip_last_error": (C.c_char_p, []),
    "sofie_hip_abi_version": (C.c_int, []),
    "sofie_hip_arena_create": (C.c_int, [_P, C.c_size_t, C.c_size_t]),
    "sofie_hip_arena_adopt": (C.c_int, [_P, _P, C.c_size_t]),
    "sofie_hip_arena_ptr": (_P, [_P, C.c_size_t]),
    "sofie_hip_arena_bytes": (C.c_size_t, [_P]),
    "sofie_hip_stream": (_P, [_P]),
    "sofie_hip_upload": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "sofie_hip_download": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "sofie_hip_copy": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "sofie_hip_fill_zero": (C.c_int, [_P, _P, C.c_size_t]),
    "sofie_hip_sync": (C.c_int, [_P]),
    "sofie_hip_gemm_f32": (C.c_int, [_P, C.POINTER(GemmF32Desc)]),
    "sofie_hip_gemm_i8": (C.c_int, [_P, C.POINTER(GemmI8Desc)]),
    "sofie_hip_gemm_i8_workspace": (C.c_size_t, [C.POINTER(GemmI8Desc)]),
    "sofie_hip_transpose_i8": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "sofie_hip_gemm_fp8": (C.c_int, [_P, C.POINTER(GemmFp8Desc)]),
    "sofie_hip_quantize_fp8": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_float]),
    "sofie_hip_quantize_linear": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_float]),
    "sofie_hip_dequantize_linear_i8": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_float]),
    "sofie_hip_dequantize_linear_i32": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_float]),
    "sofie_hip_unary_f32": (C.c_int, [_P, _P, _P, C.c_size_t, C.c_int32, C.c_float]),
    "sofie_hip_add_f32": (C.c_int, [_P, C.POINTER(AddDesc)]),
    "sofie_hip_conv_f32": (C.c_int, [_P, C.POINTER(ConvDesc), _P, _P, _P, C.c_int32, C.c_float, _P, C.POINTER(PostOps), _P]),
    "sofie_hip_conv3d_f32": (C.c_int, [_P, C.POINTER(Conv3dDesc), _P, _P, _P, C.c_int32, C.c_float, _P, C.POINTER(PostOps), _P]),
    "sofie_hip_unary_chain_f32": (C.c_int, [_P, _P, _P, C.c_size_t, C.POINTER(PostOps)]),
    "sofie_hip_conv_i8": (C.c_int, [_P, C.POINTER(ConvDesc), C.POINTER(ConvI8Args)]),
    "sofie_hip_conv_i8_workspace": (C.c_size_t, [C.POINTER(ConvDesc), C.POINTER(ConvI8Args)]),
    "sofie_hip_conv_i8_column_matrix_bytes": (C.c_size_t, [C.POINTER(ConvDesc)]),
    "sofie_hip_ctx_set_option": (C.c_int, [_P, C.c_char_p, C.c_int32]),
    "sofie_hip_gemm_i8_noalloc": (C.c_int, [_P, C.POINTER(GemmI8Desc)]),
    "sofie_hip_pack_conv_weight_i8": (C.c_int, [_P, C.POINTER(ConvDesc), _P, _P]),
    "sofie_hip_global_avg_pool_f32": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32]),
    "sofie_hip_pool_f32": (C.c_int, [_P, _P, _P, _P]),
    "sofie_hip_pool3d_f32": (C.c_int, [_P, _P, _P, _P]),
    "sofie_hip_reduce_f32": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int32, C.c_int64, C.c_int32]),
    "sofie_hip_layernorm_f32": (C.c_int, [_P, _P, _P, _P, _P, C.c_int64, C.c_int32, C.c_float, _P, _P]),
    "sofie_hip_transpose_f32": (C.c_int, [_P, _P, _P, C.c_int32, _P, _P]),
    "sofie_hip_strided_gather_f32": (C.c_int, [_P, _P, _P, C.c_int32, _P, _P, C.c_int64, C.c_int64]),
    "sofie_hip_copy_rows": (C.c_int, [_P, _P, C.c_size_t, _P, C.c_size_t, C.c_size_t, C.c_size_t]),
    "sofie_hip_binary_f32": (C.c_int, [_P, _P, C.c_int32, C.c_float]),
    "sofie_hip_softmax_f32": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int32, C.c_int64, C.c_int32]),
    "sofie_hip_gemm_chain_f32": (C.c_int, [_P, _P, C.c_int32]),
    "sofie_hip_plane_sums_to_average": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, C.c_float]),
    "sofie_hip_plane_sums_take_average": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, C.c_float]),
    "sofie_hip_batchnorm_f32": (C.c_int, [_P, _P, _P, _P, _P, _P, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "sofie_hip_global_avg_pool_i8": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_float]),
    "sofie_hip_conv_weight_i8_packed_bytes": (C.c_size_t, [C.POINTER(ConvDesc)]),
    "sofie_hip_timer_start": (C.c_int, [_P]),
    "sofie_hip_timer_stop": (C.c_int, [_P, C.POINTER(C.c_float)]),
}

_lib = None


def load_library(path=None):
    """dlopen the runtime library and type every entry point; raises if it is missing."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or lib_path()
    # torch wheels carry their own copy of the HIP runtime.  When torch shares the process (the tests use
    # it to allocate device buffers) it has to initialise first, so that one runtime serves both.
    import sys
    if "torch" in sys.modules:
        sys.modules["torch"].cuda.is_available()
    if not os.path.exists(p):
        raise SofieHipError("%s is not built: run `python -c 'import __graft_entry__ as g; g.build()'`" % p)
    lib = C.CDLL(p)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if path is None:
        _lib = lib
    return lib


class Runtime:
    """One context (stream + optional arena) on one device; methods raise SofieHipError on failure."""

    def __init__(self, device=0, external_stream=None):
        self.lib = load_library()
        h = C.c_void_p()
        self._check(self.lib.sofie_hip_ctx_create(C.byref(h), device, external_stream))
        self.ctx = h

    def close(self):
        if getattr(self, "ctx", None):
            self.lib.sofie_hip_ctx_destroy(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, status):
        if status != 0:
            raise SofieHipError("sofie_hip status %d: %s" % (status, (self.lib.sofie_hip_last_error() or b"").decode()))

    def call(self, name, *args):
        self._check(getattr(self.lib, name)(self.ctx, *args))

    def set_option(self, name, value):
        """Kernel-choice override of this context (see sofie_hip_ctx_set_option)."""
        self.call("sofie_hip_ctx_set_option", name.encode(), int(value))

    def sync(self):
        self.call("sofie_hip_sync")

    def stream(self):
        return self.lib.sofie_hip_stream(self.ctx)

    def timer_start(self):
        self.call("sofie_hip_timer_start")

    def timer_stop(self):
        ms = C.c_float()
        self.call("sofie_hip_timer_stop", C.byref(ms))
        return ms.value

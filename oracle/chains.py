"""CPU chains (test infrastructure, like the rest of this folder): the benchmark models run operator by operator, unfused,
through the C restatement.  What the parity tests and the benchmark's CPU-baseline leg compare the GPU path with."""
import numpy as np

from oracle import binding as ob


def int8_mlp_oracle(x, weights, w_scales, in_scales, omp=False):
    """Per layer: QuantizeLinear -> MatMulInteger -> Relu (int32) -> DequantizeLinear, all separate."""
    h = np.ascontiguousarray(x, dtype=np.float32)
    for w, sw, sx in zip(weights, w_scales, in_scales):
        K, N = w.shape
        q = ob.quantize_linear(h, np.float32(sx))
        acc = ob.matmul_integer(q, w, M=h.shape[0], N=N, K=K, omp=omp)
        acc = np.maximum(acc, 0)
        h = ob.dequantize_linear(acc.astype(np.int32), np.float32(np.float32(sx) * np.float32(sw)))
    return h


def int8_cnn_oracle(m, x, omp=True):
    """Operator by operator on the CPU: QuantizeLinear, then per stage conv (int32) + bias + requant + Relu (NCHW),
    GlobalAveragePool on the int8 map, fp32 Gemm."""
    h = ob.quantize_linear(np.ascontiguousarray(x, dtype=np.float32), m["in_scale"])
    for cv in m["convs"]:
        h = ob.conv_i8(h, cv["W"], cv["bias"], cv["scale"], pads=cv["pads"], strides=cv["strides"], dils=cv["dils"], relu=1,
                       out=2, omp=omp)
    pooled = ob.global_avg_pool_i8(h, m["last_scale"])
    n, c = pooled.shape
    return ob.gemm_f32(pooled, m["fc_w"], m["fc_b"], M=n, N=m["fc_w"].shape[1], K=c, bias_mode=1)

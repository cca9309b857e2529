"""Oracle-side (CPU) chains that mirror the Session objects operator by operator, unfused."""
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

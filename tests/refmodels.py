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


def make_int8_cnn(batch, hw=64, channels=(3, 64, 128, 256, 256), n_out=10, seed=5200):
    """benchmark configuration 5 as model constants: Conv3x3 s1 p1 (+folded BatchNorm = per-channel scale and bias) + Relu
    per stage, GlobalAveragePool, Gemm.  int8 weights U[-127,127], inputs U(0,1)."""
    from tests import util
    convs = []
    for l in range(len(channels) - 1):
        cin, cout = channels[l], channels[l + 1]
        K = cin * 9
        W = util.int8_sym(seed + 10 * l, cout * cin * 9).reshape(cout, cin, 3, 3)
        bias = util.int32_range(seed + 10 * l + 1, cout, -3000, 3000)
        # accumulators have a spread of about 73 * 40 * sqrt(K); the scale brings them back to a spread of ~40
        scale = ((0.5 + util.uniform01(seed + 10 * l + 2, cout)) * np.float32(0.0138 / np.sqrt(K))).astype(np.float32)
        convs.append(dict(W=W, bias=bias, scale=scale, pads=(1, 1, 1, 1), strides=(1, 1), dils=(1, 1)))
    x = util.uniform01(seed + 100, batch * channels[0] * hw * hw).reshape(batch, channels[0], hw, hw)
    fc_w = util.normal(seed + 101, channels[-1] * n_out, 0.05).reshape(channels[-1], n_out)
    fc_b = util.normal(seed + 102, n_out, 0.1)
    return dict(batch=batch, in_shape=(channels[0], hw, hw), in_scale=np.float32(1.0 / 127.0), convs=convs,
                last_scale=np.float32(0.05), fc_w=fc_w, fc_b=fc_b, x=x)


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

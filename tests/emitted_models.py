"""The models that go through the C++ emitter: every golden fixture of the reference plus the benchmark
configurations this backend adds (built here as ONNX files from seeded data).  build_all() runs at build
time on the CPU: it writes the ONNX files, runs sofie_hip_emit, and compiles each emitted header together
with a tiny C harness into tests/emitted/lib<Model>.so.  The GPU tests only load those libraries."""
import json
import os
import subprocess

import numpy as np

from sofie_amd.benchsupport import onnx_write as ow
from sofie_amd.benchsupport import synthetic as util
from sofie_amd.benchsupport.models import int8_mlp, int8_cnn  # noqa: F401  (models shared with the benchmark)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
OUT = os.path.join(ROOT, "tests", "emitted")
EMIT = os.path.join(ROOT, "sofie_amd", "emit", "bin", "sofie_hip_emit")
GOLDEN = os.path.join(ROOT, "tests", "golden")


# ---- configuration models ------------------------------------------------------------------------------------

def fp32_mlp(batch=64):
    """benchmark configuration 1: Gemm(transB=1)+Relu, Gemm+Relu, Gemm; 784 -> 128 -> 64 -> 10; W ~ N(0, 0.05), biases 0."""
    dims = [784, 128, 64, 10]
    init, nodes, x = {}, [], "X"
    for l in range(3):
        init["W%d" % l] = util.normal(1001 + l, dims[l + 1] * dims[l], 0.05).reshape(dims[l + 1], dims[l])
        init["B%d" % l] = np.zeros(dims[l + 1], dtype=np.float32)
        y = "G%d" % l
        nodes.append(ow.node("Gemm", [x, "W%d" % l, "B%d" % l], [y], alpha=1.0, beta=1.0, transB=1))
        if l < 2:
            nodes.append(ow.node("Relu", [y], ["R%d" % l]))
            y = "R%d" % l
        x = y
    X = util.uniform01(2001, batch * 784).reshape(batch, 784)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 784])], outputs=[(x, np.float32, [batch, 10])], init=init, feeds=[X])


def fp32_cnn(batch=2):
    """A small fp32 form of benchmark configuration 5: 2 x [Conv3x3 s1 p1 + Relu], GlobalAveragePool, Gemm."""
    init = {"W0": util.normal(5101, 8 * 3 * 9, 0.2).reshape(8, 3, 3, 3), "B0": util.normal(5102, 8, 0.1),
            "W1": util.normal(5103, 16 * 8 * 9, 0.1).reshape(16, 8, 3, 3), "B1": util.normal(5104, 16, 0.1),
            "WF": util.normal(5105, 16 * 10, 0.3).reshape(16, 10), "BF": util.normal(5106, 10, 0.1)}
    nodes = [ow.node("Conv", ["X", "W0", "B0"], ["C0"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("Relu", ["C0"], ["R0"]),
             ow.node("Conv", ["R0", "W1", "B1"], ["C1"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("Relu", ["C1"], ["R1"]),
             ow.node("GlobalAveragePool", ["R1"], ["P"]),
             ow.node("Gemm", ["P2", "WF", "BF"], ["Y"], alpha=1.0, beta=1.0)]
    # GlobalAveragePool gives [N,16,1,1]; the Gemm reads it as [N,16]: same bytes, so the model feeds P straight in
    nodes[-1] = ow.node("Gemm", ["P", "WF", "BF"], ["Y"], alpha=1.0, beta=1.0)
    X = util.uniform01(5001, batch * 3 * 12 * 12).reshape(batch, 3, 12, 12)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 3, 12, 12])], outputs=[("Y", np.float32, [batch, 10])], init=init, feeds=[X])


def conv_batchnorm_relu(batch=2):
    """Conv 3x3 -> BatchNormalization (kept at run time) -> Relu -> GlobalAveragePool: a model whose normalisation
    arrives un-folded."""
    init = {"W": util.normal(6101, 8 * 3 * 9, 0.3).reshape(8, 3, 3, 3),
            "gamma": (0.5 + util.uniform01(6102, 8)).astype(np.float32), "beta": util.normal(6103, 8, 0.2),
            "mean": util.normal(6104, 8, 0.5), "var": (0.2 + util.uniform01(6105, 8)).astype(np.float32)}
    nodes = [ow.node("Conv", ["X", "W"], ["C"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("BatchNormalization", ["C", "gamma", "beta", "mean", "var"], ["N"], epsilon=1e-3),
             ow.node("Relu", ["N"], ["R"]),
             ow.node("GlobalAveragePool", ["R"], ["Y"])]
    X = util.normal(6001, batch * 3 * 10 * 10).reshape(batch, 3, 10, 10)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 3, 10, 10])], outputs=[("Y", np.float32, [batch, 8, 1, 1])], init=init, feeds=[X])


def conv_pool_stack(batch=2):
    """Conv 3x3 -> Relu -> MaxPool 3x3 / stride 2 / pad 1 (the stem of a residual network) -> AveragePool 2x2 / stride 2 with
    ceil_mode over an odd image (the last window hangs over the edge) -> Flatten -> Gemm."""
    init = {"W": util.normal(6201, 6 * 3 * 9, 0.3).reshape(6, 3, 3, 3), "b": util.normal(6202, 6, 0.1),
            "F": util.normal(6203, 6 * 3 * 3 * 5, 0.2).reshape(54, 5), "c": util.normal(6204, 5, 0.1)}
    nodes = [ow.node("Conv", ["X", "W", "b"], ["C"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("Relu", ["C"], ["R"]),
             ow.node("MaxPool", ["R"], ["M"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2]),
             ow.node("AveragePool", ["M"], ["A"], kernel_shape=[2, 2], strides=[2, 2], ceil_mode=1),
             ow.node("Flatten", ["A"], ["L"], axis=1),
             ow.node("Gemm", ["L", "F", "c"], ["Y"])]
    X = util.normal(6205, batch * 3 * 10 * 10).reshape(batch, 3, 10, 10)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 3, 10, 10])], outputs=[("Y", np.float32, [batch, 5])], init=init, feeds=[X])


def classifier_head(batch=4):
    """Gemm -> Relu -> Gemm -> Softmax over the classes, and a LogSoftmax of the same logits as a second output."""
    init = {"W1": util.normal(6301, 20 * 32, 0.2).reshape(20, 32), "b1": util.normal(6302, 32, 0.1),
            "W2": util.normal(6303, 32 * 7, 0.3).reshape(32, 7), "b2": util.normal(6304, 7, 0.1)}
    nodes = [ow.node("Gemm", ["X", "W1", "b1"], ["H"]), ow.node("Relu", ["H"], ["R"]), ow.node("Gemm", ["R", "W2", "b2"], ["L"]),
             ow.node("Softmax", ["L"], ["P"], axis=1), ow.node("LogSoftmax", ["L"], ["Q"], axis=-1)]
    X = util.normal(6305, batch * 20).reshape(batch, 20)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 20])], outputs=[("P", np.float32, [batch, 7]), ("Q", np.float32, [batch, 7])], init=init,
                feeds=[X])


def gemm_chain_widths(batch=64):
    """X[64,32] -> Gemm(128) -> Gemm(64) -> Gemm(96) -> Softmax: three products of different widths that the generator hands to the
    runtime as one call; planned by per-operator lifetimes, the third output would take the start of the first one's memory with a
    different row pitch."""
    init = {"W0": util.normal(6401, 32 * 128, 0.2).reshape(32, 128), "b0": util.normal(6402, 128, 0.1),
            "W1": util.normal(6403, 128 * 64, 0.1).reshape(128, 64), "b1": util.normal(6404, 64, 0.1),
            "W2": util.normal(6405, 64 * 96, 0.1).reshape(64, 96), "b2": util.normal(6406, 96, 0.1)}
    nodes = [ow.node("Gemm", ["X", "W0", "b0"], ["Y0"]), ow.node("Gemm", ["Y0", "W1", "b1"], ["Y1"]), ow.node("Gemm", ["Y1", "W2", "b2"], ["Y2"]),
             ow.node("Softmax", ["Y2"], ["P"], axis=1)]
    X = util.normal(6407, batch * 32).reshape(batch, 32)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 32])], outputs=[("P", np.float32, [batch, 96])], init=init, feeds=[X])


def shape_plumbing(batch=3):
    """Reshape (with 0 and -1), Transpose, Squeeze / Unsqueeze (axes as input and as attribute), Concat and Flatten around a Gemm:
    X [b, 2, 3, 4] -> Transpose(0, 2, 1, 3) -> Reshape [0, 3, -1] -> Concat with Z [b, 3, 2] along the last axis -> Unsqueeze(1) -> Squeeze(1)
    -> Flatten -> Gemm."""
    init = {"shape": np.array([0, 3, -1], np.int64), "ax1": np.array([1], np.int64), "W": util.normal(6401, 30 * 6, 0.2).reshape(30, 6),
            "b": util.normal(6402, 6, 0.1)}
    nodes = [ow.node("Transpose", ["X"], ["T"], perm=[0, 2, 1, 3]), ow.node("Reshape", ["T", "shape"], ["R"]),
             ow.node("Concat", ["R", "Z"], ["C"], axis=-1), ow.node("Unsqueeze", ["C", "ax1"], ["U"]), ow.node("Squeeze", ["U"], ["S"], axes=[1]),
             ow.node("Flatten", ["S"], ["F"], axis=1), ow.node("Gemm", ["F", "W", "b"], ["Y"])]
    X = util.normal(6403, batch * 24).reshape(batch, 2, 3, 4)
    Z = util.normal(6404, batch * 6).reshape(batch, 3, 2)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 2, 3, 4]), ("Z", np.float32, [batch, 3, 2])], outputs=[("Y", np.float32, [batch, 6])],
                init=init, feeds=[X, Z])


def layernorm_block(batch=3):
    """Gemm -> LayerNormalization over the features (with its Mean as a second output) -> Gelu -> Gemm: the shape of a transformer's feed-forward entry."""
    init = {"W1": util.normal(6501, 12 * 16, 0.3).reshape(12, 16), "b1": util.normal(6502, 16, 0.1), "g": (1 + 0.2 * util.normal(6503, 16)).astype(np.float32),
            "beta": util.normal(6504, 16, 0.1), "W2": util.normal(6505, 16 * 4, 0.3).reshape(16, 4)}
    nodes = [ow.node("Gemm", ["X", "W1", "b1"], ["H"]), ow.node("LayerNormalization", ["H", "g", "beta"], ["N", "M"], axis=-1, epsilon=1e-5),
             ow.node("Gelu", ["N"], ["A"]), ow.node("MatMul", ["A", "W2"], ["Y"])]
    X = util.normal(6506, batch * 12).reshape(batch, 12)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 12])], outputs=[("Y", np.float32, [batch, 4]), ("M", np.float32, [batch, 1])], init=init, feeds=[X])


def reduce_block(batch=3, named=None):
    """ReduceMean over the last axis (kept) -> Sub (centring) -> ReduceL2 with the axes as an input; a ReduceMax over the middle axis and a ReduceSum
    over the batch itself as further outputs.  `named` leaves the batch as a run-time parameter."""
    b = named if named else batch
    init = {"ax": np.array([-1], np.int64)}
    nodes = [ow.node("ReduceMean", ["X"], ["M"], axes=[2], keepdims=1), ow.node("Sub", ["X", "M"], ["C"]),
             ow.node("ReduceL2", ["C", "ax"], ["Y1"], keepdims=0), ow.node("ReduceMax", ["X"], ["Y2"], axes=[1], keepdims=0),
             ow.node("ReduceSum", ["X"], ["Y3"], axes=[0], keepdims=1)]
    X = (util.normal(6601, batch * 24) + np.float32(0.25)).reshape(batch, 4, 6)
    return dict(nodes=nodes, inputs=[("X", np.float32, [b, 4, 6])], outputs=[("Y1", np.float32, [b, 4]), ("Y2", np.float32, [b, 6]), ("Y3", np.float32, [1, 4, 6])],
                init=init, feeds=[X])


def hard_activations(batch=4):
    """Gemm -> HardSwish -> Gemm -> Swish -> HardSigmoid (non-default alpha / beta), and a Conv -> HardSwish on a second input: every one of them
    rides in the store of the product before it."""
    init = {"W1": util.normal(6701, 12 * 24, 0.6).reshape(12, 24), "b1": util.normal(6702, 24, 0.5), "W2": util.normal(6703, 24 * 5, 0.5).reshape(24, 5),
            "b2": util.normal(6704, 5, 0.3), "K": util.normal(6705, 4 * 3 * 3 * 3, 0.5).reshape(4, 3, 3, 3)}
    nodes = [ow.node("Gemm", ["X", "W1", "b1"], ["H"]), ow.node("HardSwish", ["H"], ["A"]), ow.node("Gemm", ["A", "W2", "b2"], ["L"]),
             ow.node("Swish", ["L"], ["S"]), ow.node("HardSigmoid", ["S"], ["Y"], alpha=0.25, beta=0.4),
             ow.node("Conv", ["Z", "K"], ["C"], kernel_shape=[3, 3], pads=[1, 1, 1, 1]), ow.node("HardSwish", ["C"], ["V"])]
    X, Z = util.normal(6706, batch * 12, 1.5).reshape(batch, 12), util.normal(6707, batch * 3 * 6 * 6, 1.5).reshape(batch, 3, 6, 6)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 12]), ("Z", np.float32, [batch, 3, 6, 6])],
                outputs=[("Y", np.float32, [batch, 5]), ("V", np.float32, [batch, 4, 6, 6])], init=init, feeds=[X, Z])


def indexing_block(batch=3, named=None):
    """Split of [b, 6, 8] along the last axis into 3 + 3 + 2 columns (no sizes given: the last part is the short one), a Slice that walks the middle axis
    backwards in steps of 2, a Gather of three rows (one counted from the end), a Tile of a part and an Expand of a gathered row; four outputs."""
    b = named if named else batch
    i64 = lambda *v: np.array(v, np.int64)
    init = {"st": i64(-1, 1), "en": i64(-100, 7), "ax": i64(1, 2), "sp": i64(-2, 1), "idx": i64(4, -1, 0), "rep": i64(1, 2, 3), "one": i64(2), "shape": i64(1, 5, 8)}
    nodes = [ow.node("Split", ["X"], ["A", "B", "Cc"], axis=-1), ow.node("Slice", ["X", "st", "en", "ax", "sp"], ["S"]),
             ow.node("Gather", ["X", "idx"], ["G"], axis=1), ow.node("Tile", ["Cc", "rep"], ["T"]),
             ow.node("Gather", ["X", "one"], ["R"], axis=1), ow.node("Expand", ["R", "shape"], ["E"]), ow.node("Add", ["A", "B"], ["AB"])]
    X = util.normal(6801, batch * 48).reshape(batch, 6, 8)
    return dict(nodes=nodes, inputs=[("X", np.float32, [b, 6, 8])],
                outputs=[("AB", np.float32, [b, 6, 3]), ("S", np.float32, [b, 3, 6]), ("G", np.float32, [b, 3, 8]), ("T", np.float32, [b, 12, 6]), ("E", np.float32, [b, 5, 8])],
                init=init, feeds=[X])


def softmax_head(batch=4):
    """Gemm -> Softmax over the classes (one output)."""
    spec = classifier_head(batch)
    return dict(spec, nodes=[spec["nodes"][0], spec["nodes"][1], spec["nodes"][2], spec["nodes"][3]], outputs=[spec["outputs"][0]])


def qlinear_matmul_relu(M=16, K=64, N=48):
    """QuantizeLinear -> QLinearMatMul (per-column weight scales) -> Relu (int8) -> DequantizeLinear."""
    W = util.int8_sym(7101, K * N).reshape(K, N)
    sx, sy = np.float32(0.02), np.float32(0.05)
    sw = ((0.5 + util.uniform01(7102, N)) * np.float32(sy / (sx * 73.0 * np.sqrt(K)))).astype(np.float32)
    init = {"W": W, "sx": np.array(sx, np.float32), "sw": sw, "sy": np.array(sy, np.float32), "zp": np.zeros((), np.int8)}
    nodes = [ow.node("QuantizeLinear", ["X", "sx", "zp"], ["Q"]),
             ow.node("QLinearMatMul", ["Q", "sx", "zp", "W", "sw", "zp", "sy", "zp"], ["P"]),
             ow.node("Relu", ["P"], ["R"]),
             ow.node("DequantizeLinear", ["R", "sy", "zp"], ["Y"])]
    X = util.normal(7001, M * K).reshape(M, K)
    mult = ((sx * sw).astype(np.float32) / sy).astype(np.float32)
    return dict(nodes=nodes, inputs=[("X", np.float32, [M, K])], outputs=[("Y", np.float32, [M, N])], init=init, feeds=[X],
                consts=dict(W=W, sx=sx, sy=sy, mult=mult))


def conv_integer_dequantize(batch=2):
    """QuantizeLinear -> ConvInteger (int32 accumulators out) -> Relu -> DequantizeLinear(int32)."""
    W = util.int8_sym(7201, 6 * 4 * 9).reshape(6, 4, 3, 3)
    sx = np.float32(0.03)
    sacc = np.float32(sx * 0.01)
    init = {"W": W, "sx": np.array(sx, np.float32), "sacc": np.array(sacc, np.float32), "zp": np.zeros((), np.int8)}
    nodes = [ow.node("QuantizeLinear", ["X", "sx", "zp"], ["Q"]),
             ow.node("ConvInteger", ["Q", "W", "zp", "zp"], ["A"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("Relu", ["A"], ["R"]),
             ow.node("DequantizeLinear", ["R", "sacc"], ["Y"])]
    X = util.normal(7202, batch * 4 * 7 * 7).reshape(batch, 4, 7, 7)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 4, 7, 7])], outputs=[("Y", np.float32, [batch, 6, 7, 7])], init=init,
                feeds=[X], consts=dict(W=W, sx=sx, sacc=sacc))


def with_named_batch(spec, param="N"):
    """The same graph with the leading dimension of every input and output left as a named parameter."""
    spec = dict(spec)
    spec["inputs"] = [(n, dt, [param] + list(sh[1:])) for n, dt, sh in spec["inputs"]]
    spec["outputs"] = [(n, dt, [param] + list(sh[1:])) for n, dt, sh in spec["outputs"]]
    return spec


def dynamic_linear():
    """Gemm + Relu with the batch as a run-time parameter: the weights of the reference's own test
    (tests/alpaka/TestAlpakaLinear.cxx:121-159)."""
    W = np.array([[0.5, -1.0, 0.25], [0.75, 0.5, -0.5], [-0.25, 1.0, 0.75], [1.5, -0.75, 0.5]], np.float32)
    B = np.array([0.5, -0.5, 0.25], np.float32)
    nodes = [ow.node("Gemm", ["X", "W", "B"], ["G"]), ow.node("Relu", ["G"], ["Y"])]
    return dict(nodes=nodes, inputs=[("X", np.float32, ["N", 4])], outputs=[("Y", np.float32, ["N", 3])], init={"W": W, "B": B},
                consts=dict(W=W, B=B))


def dynamic_matmul_batched():
    """A[N,4,8] x B[N,8,6], both operands carrying the run-time batch (tests/alpaka/TestAlpakaLinear.cxx:161-210)."""
    nodes = [ow.node("MatMul", ["A", "B"], ["Y"])]
    return dict(nodes=nodes, inputs=[("A", np.float32, ["N", 4, 8]), ("B", np.float32, ["N", 8, 6])],
                outputs=[("Y", np.float32, ["N", 4, 6])], init={})


def elementwise_chains(batch=6):
    """One-to-one operators behind a Gemm, behind a Conv and behind a graph input: the generator folds them into the
    producer's store (its own activation + at most four further links) or into one pass over the data."""
    W = (util.normal(7401, 20 * 12) * np.float32(0.3)).reshape(20, 12)
    B = util.normal(7402, 12) * np.float32(0.1)
    Wc = (util.normal(7403, 5 * 3 * 9) * np.float32(0.2)).reshape(5, 3, 3, 3)
    init = {"W": W, "B": B, "Wc": Wc, "lo": np.array(0.5, np.float32), "hi": np.array(3.0, np.float32)}
    nodes = [
        # Gemm -> LeakyRelu (the Gemm's activation) -> Exp -> Clip -> Sqrt -> Log (four links) -> Neg (one more pass)
        ow.node("Gemm", ["X", "W", "B"], ["g0"]), ow.node("LeakyRelu", ["g0"], ["g1"], alpha=0.1), ow.node("Exp", ["g1"], ["g2"]),
        ow.node("Clip", ["g2", "lo", "hi"], ["g3"]), ow.node("Sqrt", ["g3"], ["g4"]), ow.node("Log", ["g4"], ["g5"]),
        ow.node("Neg", ["g5"], ["Y"]),
        # Conv -> Tanh -> Abs -> Softplus -> Reciprocal
        ow.node("Conv", ["I", "Wc"], ["c0"], kernel_shape=[3, 3], pads=[1, 1, 1, 1]), ow.node("Tanh", ["c0"], ["c1"]),
        ow.node("Abs", ["c1"], ["c2"]), ow.node("Softplus", ["c2"], ["c3"]), ow.node("Reciprocal", ["c3"], ["Z"]),
        # a graph input through Sin -> Exp -> Atan -> Floor -> Identity -> Asinh: one chain of four, then one of two
        ow.node("Sin", ["X"], ["s0"]), ow.node("Exp", ["s0"], ["s1"]), ow.node("Atan", ["s1"], ["s2"]), ow.node("Floor", ["s2"], ["s3"]),
        ow.node("Identity", ["s3"], ["s4"]), ow.node("Asinh", ["s4"], ["V"]),
    ]
    X = util.normal(7404, batch * 20).reshape(batch, 20)
    I = util.normal(7405, 2 * 3 * 6 * 6).reshape(2, 3, 6, 6)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 20]), ("I", np.float32, [2, 3, 6, 6])],
                outputs=[("Y", np.float32, [batch, 12]), ("Z", np.float32, [2, 5, 6, 6]), ("V", np.float32, [batch, 20])], init=init, feeds=[X, I])


def dynamic_residual():
    """Run-time batch through a broadcasting Add: Y = Relu(X * W + Z) + b with X[N,6], Z[N,5] both batched and b[5] broadcast."""
    W = (util.normal(7501, 6 * 5) * np.float32(0.4)).reshape(6, 5)
    b = util.normal(7502, 5)
    nodes = [ow.node("MatMul", ["X", "W"], ["P"]), ow.node("Add", ["P", "Z"], ["S"]), ow.node("Relu", ["S"], ["R"]), ow.node("Add", ["b", "R"], ["Y"])]
    return dict(nodes=nodes, inputs=[("X", np.float32, ["N", 6]), ("Z", np.float32, ["N", 5])], outputs=[("Y", np.float32, ["N", 5])],
                init={"W": W, "b": b}, consts=dict(W=W, b=b))


def residual_block(batch=2):
    """Conv -> Add(shortcut) -> Relu -> GlobalAveragePool -> Flatten -> Gemm -> Add(second input) -> Sigmoid: both Adds have
    operands of equal shape, so each joins the store of the operator before it, ahead of the activation."""
    Wc = (util.normal(7601, 8 * 8 * 9) * np.float32(0.15)).reshape(8, 8, 3, 3)
    Bc = util.normal(7602, 8) * np.float32(0.1)
    W = (util.normal(7603, 8 * 4) * np.float32(0.5)).reshape(8, 4)
    b = util.normal(7604, 4) * np.float32(0.2)
    nodes = [ow.node("Conv", ["X", "Wc", "Bc"], ["c0"], kernel_shape=[3, 3], pads=[1, 1, 1, 1]), ow.node("Add", ["c0", "X"], ["s0"]),
             ow.node("Relu", ["s0"], ["r0"]), ow.node("GlobalAveragePool", ["r0"], ["p"]), ow.node("Flatten", ["p"], ["f"], axis=1),
             ow.node("Gemm", ["f", "W", "b"], ["g"]), ow.node("Add", ["Z", "g"], ["s1"]), ow.node("Sigmoid", ["s1"], ["Y"])]
    X = util.normal(7605, batch * 8 * 6 * 6).reshape(batch, 8, 6, 6)
    Z = util.normal(7606, batch * 4).reshape(batch, 4)
    return dict(nodes=nodes, inputs=[("X", np.float32, [batch, 8, 6, 6]), ("Z", np.float32, [batch, 4])], outputs=[("Y", np.float32, [batch, 4])],
                init={"Wc": Wc, "Bc": Bc, "W": W, "b": b}, feeds=[X, Z])


def parse_rewrites():
    """What the reference's parser rewrites before any operator is built (parsers/src/RModelParser_ONNX.cxx:1116-1140, 1186-1207) and
    what its operators fold (ROperator_Gemm.hxx:317-373, ROperator_BasicBinary.hxx:191-257): a Cast to the same type, Transpose -> MatMul,
    MatMul + Add, Conv + Add of a one-dimensional initializer (taken as the per-channel bias), a Gemm of weights only, a sum of constants."""
    W2 = (util.normal(7701, 5 * 6) * np.float32(0.3)).reshape(5, 6)
    b1 = util.normal(7702, 5)
    W3 = (util.normal(7703, 6 * 3) * np.float32(0.3)).reshape(6, 3)
    Ka, Kb, Kc = util.normal(7704, 8).reshape(4, 2), util.normal(7705, 6).reshape(2, 3), util.normal(7706, 12).reshape(4, 3)
    Kbt, Kd = np.ascontiguousarray(Kb.T), util.normal(7712, 12).reshape(4, 3)
    Wc = (util.normal(7707, 3 * 2) * np.float32(0.5)).reshape(3, 2, 1, 1)
    cb = util.normal(7708, 3)
    nodes = [
        ow.node("Cast", ["X"], ["Xc"], to=1), ow.node("Transpose", ["W2"], ["Wt"], perm=[1, 0]), ow.node("MatMul", ["Xc", "Wt"], ["m1"]),
        ow.node("Add", ["m1", "b1"], ["Y1"]),
        ow.node("Transpose", ["A2"], ["At"]), ow.node("MatMul", ["At", "W3"], ["m2"]),
        ow.node("Gemm", ["Ka", "Kb", "Kc"], ["K"], alpha=0.5, beta=2.0), ow.node("Relu", ["K"], ["Kr"]),       # folded, Relu included
        ow.node("Gemm", ["Ka", "Kbt", "Kd"], ["K2"], transB=1), ow.node("Add", ["Kr", "K2"], ["Ks"]),             # a sum of two folded products
        ow.node("Add", ["m2", "Ks"], ["Y2"]),
        ow.node("Conv", ["I", "Wc"], ["c"], kernel_shape=[1, 1], pads=[0, 0, 0, 0]), ow.node("Add", ["c", "cb"], ["Y3"]),
    ]
    X, A2, I = util.normal(7709, 24).reshape(4, 6), util.normal(7710, 24).reshape(6, 4), util.normal(7711, 18).reshape(1, 2, 3, 3)
    # expected values, straight from the definitions (the Conv + Add as the reference reads it: one bias per channel)
    Ks = np.maximum(0.5 * (Ka.astype(np.float64) @ Kb) + 2.0 * Kc, 0) + (Ka.astype(np.float64) @ Kb + Kd)
    want = [X.astype(np.float64) @ W2.T + b1, A2.T.astype(np.float64) @ W3 + Ks,
            np.einsum("nchw,oc->nohw", I.astype(np.float64), Wc[:, :, 0, 0]) + cb.reshape(1, 3, 1, 1)]
    return dict(nodes=nodes, inputs=[("X", np.float32, [4, 6]), ("A2", np.float32, [6, 4]), ("I", np.float32, [1, 2, 3, 3])],
                outputs=[("Y1", np.float32, [4, 5]), ("Y2", np.float32, [4, 3]), ("Y3", np.float32, [1, 3, 3, 3])],
                init={"W2": W2, "b1": b1, "W3": W3, "Ka": Ka, "Kb": Kb, "Kbt": Kbt, "Kc": Kc, "Kd": Kd, "Wc": Wc, "cb": cb}, feeds=[X, A2, I], want=want)


# Models of the reference's own tests whose expected outputs are literals in those tests (tests/cpu/TestCustomModelsFromONNX.cxx:509-527,
# 1672-1700; the graphs are those of tests/models/generators/generate_input_models.py:1795-1838, 3411-3464, restated here as data).
def reference_constant_folding_cases():
    f = np.float32
    return {
        "Gemm_ConstantFolding": dict(
            nodes=[ow.node("Gemm", ["A", "B", "C"], ["Y"], alpha=1.0, beta=1.0, transA=0, transB=0)], inputs=[], outputs=[("Y", f, [2, 2])],
            init={"A": np.array([[1, 2, 3], [4, 5, 6]], f), "B": np.array([[7, 8], [9, 10], [11, 12]], f), "C": np.ones((2, 2), f)},
            feeds=[], want=[[59, 65, 140, 155]]),
        "Gemm_ConstantFolding_Shared": dict(
            nodes=[ow.node("Gemm", ["A1", "B", "C1"], ["Y1"], alpha=1.0, beta=1.0, transA=0, transB=0),
                   ow.node("Gemm", ["A2", "B", "C2"], ["Y2"], alpha=1.0, beta=1.0, transA=0, transB=0)],
            inputs=[("A2", f, [2, 2])], outputs=[("Y1", f, [2, 2]), ("Y2", f, [2, 2])],
            init={"A1": np.array([[1, 2], [3, 4]], f), "B": np.eye(2, dtype=f), "C1": np.ones((2, 2), f), "C2": np.full((2, 2), 10, f)},
            feeds=[np.array([[5, 6], [7, 8]], f)], want=[[2, 3, 4, 5], [15, 16, 17, 18]]),
        "MatMul_1D_Constant": dict(
            nodes=[ow.node("MatMul", ["A", "B"], ["Y"])], inputs=[], outputs=[("Y", f, [2])],
            init={"A": np.array([1, 2, 3], f), "B": np.array([[1, 2], [3, 4], [5, 6]], f)}, feeds=[], want=[[22, 28]]),
    }


def reference_stacked_matmul_cases():
    f = np.float32
    return {
        "MatMul_Stacked": dict(nodes=[ow.node("MatMul", ["input1", "input2"], ["output"])], inputs=[("input1", f, ["N", 2, 2]), ("input2", f, [2, 1])],
                               outputs=[("output", f, ["N", 2, 1])], init={}, feeds=[np.arange(1, 9, dtype=f), np.array([2, 3], f)], want=[8, 18, 28, 38]),
        "MatMul_Stacked2": dict(nodes=[ow.node("MatMul", ["input1", "input2"], ["output"])], inputs=[("input1", f, ["N", 2, 2]), ("input2", f, ["N", 2, 1])],
                                outputs=[("output", f, ["N", 2, 1])], init={}, feeds=[np.arange(1, 9, dtype=f), np.array([2, 3, 3, 2], f)], want=[8, 18, 27, 37]),
    }


DYNAMIC_MODELS = {    "Dynamic_ResidualBlock": lambda: with_named_batch(residual_block(2), "N"),
    "DynamicResidual": dynamic_residual,

    "DynamicLinear": dynamic_linear,
    "DynamicMatMulBatched": dynamic_matmul_batched,
    "Dynamic_int8_MLP": lambda: with_named_batch(int8_mlp([64, 128, 96, 32], 48), "batch_size"),
    "Dynamic_int8_CNN": lambda: with_named_batch(int8_cnn(2, 12), "N"),
    "Dynamic_ConvBatchNormRelu": lambda: with_named_batch(conv_batchnorm_relu(2), "bs"),
    "Dynamic_ConvPoolStack": lambda: with_named_batch(conv_pool_stack(2), "N"),
    "Dynamic_SoftmaxHead": lambda: with_named_batch(softmax_head(4), "N"),
    "Dynamic_ShapePlumbing": lambda: with_named_batch(shape_plumbing(3), "N"),
    "Dynamic_ReduceBlock": lambda: reduce_block(3, "N"),
    "Dynamic_IndexingBlock": lambda: indexing_block(3, "N"),
    "Dynamic_int8_CNN_plane_sums": lambda: with_named_batch(int8_cnn(2, 16, (3, 64, 128)), "N"),
}

CONFIG_MODELS = {
    "ResidualBlock": lambda: residual_block(2),
    "QLinearMatMulRelu": lambda: qlinear_matmul_relu(),
    "ConvIntegerDequantize": lambda: conv_integer_dequantize(),
    "ConvBatchNormRelu": lambda: conv_batchnorm_relu(2),
    "ConvPoolStack": lambda: conv_pool_stack(2),
    "ShapePlumbing": lambda: shape_plumbing(3),
    "Config5_int8_CNN_small": lambda: int8_cnn(2, 12),
    "Int8_CNN_plane_sums": lambda: int8_cnn(2, 16, (3, 64, 128)),   # planes of 256 pixels: the last convolution sums them itself
    "GemmChainWidths": lambda: gemm_chain_widths(64),
    "Config1_fp32_MLP": lambda: fp32_mlp(64),
    "Config2_int8_MLP_small": lambda: int8_mlp([64, 128, 96, 32], 48),
    "Config2_int8_MLP_mid": lambda: int8_mlp([256, 512, 512, 256], 256),
}


def golden_models():
    return sorted(json.load(open(os.path.join(GOLDEN, "fixtures.json"))).keys())


# ---- build ----------------------------------------------------------------------------------------------------

HARNESS = r'''
#include "%(model)s_GPU_HIP.hxx"
#include <cstring>
// C harness around the emitted Session for the Python tests: returns 0, or 1 with the exception text in err.
extern "C" int run_model(const char *weights, const float *const *inputs, float *output, unsigned long output_len, char *err, int errlen)
{
   try {
      SOFIE_%(model)s::Session s(weights);
      auto y = s.infer(%(args)s);
      if (y.size() != output_len)
         throw std::runtime_error("output has " + std::to_string(y.size()) + " elements");
      std::memcpy(output, y.data(), y.size() * sizeof(float));
      // a second inference on the same session must give the same answer (the pool is reused)
      auto y2 = s.infer(%(args)s);
      if (std::memcmp(y.data(), y2.data(), y.size() * sizeof(float)) != 0)
         throw std::runtime_error("second inference differs from the first");
      return 0;
   } catch (const std::exception &e) {
      std::strncpy(err, e.what(), errlen - 1);
      err[errlen - 1] = 0;
      return 1;
   }
}
// The same inference on device memory of the caller, through infer(std::span<ViewConstF1D const>, std::span<ViewF1D>).
// The caller's memory is the arena of a second context; `misalign` (in floats) moves every view off the 256-byte boundary,
// which makes the Session copy through its own regions instead of working in place.
extern "C" int run_model_views(const char *weights, const float *const *inputs, const unsigned long *input_lens, int n_inputs, float *output,
                               unsigned long output_len, int misalign, char *err, int errlen)
{
   sofie_hip_ctx *helper = nullptr;
   int rc = 0;
   try {
      using namespace SOFIE_%(model)s;
      std::size_t total = 4096;
      for (int i = 0; i < n_inputs; ++i)
         total += (input_lens[i] * sizeof(float) + 511) / 256 * 256;
      total += (output_len * sizeof(float) + 511) / 256 * 256;
      if (sofie_hip_ctx_create(&helper, 0, nullptr) || sofie_hip_arena_create(helper, total, 256))
         throw std::runtime_error(sofie_hip_last_error());
      char *base = static_cast<char *>(sofie_hip_arena_ptr(helper, 0));
      std::size_t off = 0;
      std::vector<ViewConstF1D> in;
      for (int i = 0; i < n_inputs; ++i) {
         float *p = reinterpret_cast<float *>(base + off) + misalign;
         detail::Check(sofie_hip_upload(helper, p, inputs[i], input_lens[i] * sizeof(float)), "upload");
         in.push_back(ViewConstF1D{p, input_lens[i]});
         off += (input_lens[i] * sizeof(float) + 511) / 256 * 256;
      }
      float *out = reinterpret_cast<float *>(base + off) + misalign;
      detail::Check(sofie_hip_fill_zero(helper, out, output_len * sizeof(float)), "clear");
      detail::Check(sofie_hip_sync(helper), "upload");
      std::vector<ViewF1D> outs{ViewF1D{out, output_len}};
      Session s(weights);
      s.infer(std::span<ViewConstF1D const>(in), std::span<ViewF1D>(outs));
      detail::Check(sofie_hip_download(helper, output, out, output_len * sizeof(float)), "download");
      detail::Check(sofie_hip_sync(helper), "download");
      // a view that is too small is refused before anything runs
      outs[0].size = output_len - 1;
      bool threw = false;
      try {
         s.infer(std::span<ViewConstF1D const>(in), std::span<ViewF1D>(outs));
      } catch (const std::runtime_error &) {
         threw = true;
      }
      if (!threw)
         throw std::runtime_error("a short output view was accepted");
   } catch (const std::exception &e) {
      std::strncpy(err, e.what(), errlen - 1);
      err[errlen - 1] = 0;
      rc = 1;
   }
   if (helper)
      sofie_hip_ctx_destroy(helper);
   return rc;
}
extern "C" unsigned long arena_bytes() { return SOFIE_%(model)s::Session::kArenaBytes; }
extern "C" unsigned long pool_bytes() { return SOFIE_%(model)s::Session::kIntermediatePoolBytes; }
'''


# Sessions with a run-time batch: kept open across calls so that a test can change the batch between inferences.
DYNAMIC_HARNESS = r'''
#include "%(model)s_GPU_HIP.hxx"
#include <cstring>
using Session = SOFIE_%(model)s::Session;
static int fail(char *err, int errlen, const char *what)
{
   std::strncpy(err, what, errlen - 1);
   err[errlen - 1] = 0;
   return 1;
}
static void flatten(const std::vector<float> &y, std::vector<float> &all) { all.insert(all.end(), y.begin(), y.end()); }
[[maybe_unused]] static void flatten(const std::vector<std::vector<float>> &ys, std::vector<float> &all)
{
   for (auto &y : ys)
      flatten(y, all);
}
extern "C" void *dyn_open(const char *weights, unsigned long max_batch, char *err, int errlen)
{
   try {
      return new Session(weights, max_batch);
   } catch (const std::exception &e) {
      fail(err, errlen, e.what());
      return nullptr;
   }
}
extern "C" void dyn_close(void *s) { delete static_cast<Session *>(s); }
extern "C" long dyn_infer(void *s, unsigned long batch, const float *const *inputs, float *output, unsigned long capacity, char *err, int errlen)
{
   try {
      std::vector<float> y;
      flatten(static_cast<Session *>(s)->infer(batch, %(args)s), y);      // several outputs come back one after the other
      if (y.size() > capacity)
         throw std::runtime_error("output has " + std::to_string(y.size()) + " elements");
      std::memcpy(output, y.data(), y.size() * sizeof(float));
      return (long)y.size();
   } catch (const std::exception &e) {
      fail(err, errlen, e.what());
      return -1;
   }
}
extern "C" int dyn_maintenance(void *s, int what, char *err, int errlen)
{
   try {
      if (what == 0)
         static_cast<Session *>(s)->resetState();
      else
         static_cast<Session *>(s)->SetWeightsToZero();
      return 0;
   } catch (const std::exception &e) {
      return fail(err, errlen, e.what());
   }
}
extern "C" double pool_statistics(void *s, unsigned long *free_bytes, unsigned long *largest)
{
   *free_bytes = static_cast<Session *>(s)->GetTotalFreeMemory();
   *largest = static_cast<Session *>(s)->GetLargestFreeBlock();
   return static_cast<Session *>(s)->GetFragmentation();
}
static_assert(SOFIE_%(model)s::inputTensorDims.size() >= 1 && SOFIE_%(model)s::hasDynamicInputTensors &&
              SOFIE_%(model)s::inputTensorDims[0].data[0].kind == SOFIE_%(model)s::SingleDim::Kind::Symbolic,
              "the leading dimension of the first input is the run-time parameter");
extern "C" unsigned long arena_bytes(unsigned long max_batch) { return Session::ArenaBytes(max_batch); }
extern "C" unsigned long pool_bytes(void *s) { return static_cast<Session *>(s)->GetIntermediateMemoryPoolSize(); }
'''


# a model with several float outputs: infer returns std::vector<std::vector<float>>, handed back concatenated
MULTI_OUTPUT_HARNESS = r'''
#include "%(model)s_GPU_HIP.hxx"
#include <cstring>
static void flatten(const std::vector<float> &y, std::vector<float> &all) { all.insert(all.end(), y.begin(), y.end()); }
static void flatten(const std::vector<std::vector<float>> &ys, std::vector<float> &all)
{
   for (auto &y : ys)
      flatten(y, all);
}
extern "C" int run_model(const char *weights, const float *const *inputs, float *output, unsigned long output_len, char *err, int errlen)
{
   (void)inputs;
   try {
      SOFIE_%(model)s::Session s(weights);
      std::vector<float> all;
      flatten(s.infer(%(args)s), all);
      if (all.size() != output_len)
         throw std::runtime_error("outputs have " + std::to_string(all.size()) + " elements");
      std::memcpy(output, all.data(), all.size() * sizeof(float));
      return 0;
   } catch (const std::exception &e) {
      std::strncpy(err, e.what(), errlen - 1);
      err[errlen - 1] = 0;
      return 1;
   }
}
'''


# Benchmark harness around the emitted Session of the int8 MLP at its full size: the Session lives across calls, the input
# stays resident on the device, and the timed region is the reference benchmark's (benchmark/src/BenchmarkEmitter.cxx.in:486-504):
# N x infer_nosync, one wait, wall clock.
def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return r.stdout


API_MODELS = ("ApiGemmRelu", "ApiFp8Gemm")


def emit_and_compile(model, onnx_path, n_inputs, *flags):
    _run([EMIT, onnx_path, OUT] + list(flags))
    return compile_harness(model, n_inputs)


def compile_harness(model, n_inputs):
    src = os.path.join(OUT, model + "_harness.cxx")
    with open(src, "w") as f:
        f.write(HARNESS % dict(model=model, args=", ".join("inputs[%d]" % i for i in range(n_inputs))))
    return compile_shared(src, os.path.join(OUT, "lib%s.so" % model))


def emit_and_compile_dynamic(model, onnx_path, n_inputs):
    _run([EMIT, onnx_path, OUT])
    src = os.path.join(OUT, model + "_harness.cxx")
    with open(src, "w") as f:
        f.write(DYNAMIC_HARNESS % dict(model=model, args=", ".join("inputs[%d]" % i for i in range(n_inputs))))
    return compile_shared(src, os.path.join(OUT, "lib%s.so" % model))


def compile_shared(src, lib):
    _run(["g++", "-O1", "-std=c++20", "-fPIC", "-shared", "-I" + os.path.join(ROOT, "include"), "-I" + OUT, src, "-o", lib,
          "-L" + os.path.join(ROOT, "sofie_amd", "lib"), "-lsofie_hip", "-Wl,-rpath," + os.path.join(ROOT, "sofie_amd", "lib"),
          "-Wl,-rpath,$ORIGIN/../../sofie_amd/lib"])
    return lib


from sofie_amd.benchsupport.emitted import BenchSession, BENCH_MODEL, bench_mlp_spec  # noqa: F401,E402


def build_all(jobs=8):
    from concurrent.futures import ThreadPoolExecutor
    from tests import onnx_lite
    os.makedirs(OUT, exist_ok=True)
    work = []
    for m in golden_models():
        p = os.path.join(GOLDEN, "models", m + ".onnx")
        work.append((m, p, len(onnx_lite.load(p)["inputs"])))
    for m, make in CONFIG_MODELS.items():
        spec = make()
        p = os.path.join(OUT, m + ".onnx")
        ow.write(p, spec["nodes"], spec["inputs"], spec["outputs"], spec["init"], name=m)
        work.append((m, p, len(spec["inputs"])))
    # the same model with its weights in a safetensors file
    work.append(("Linear_16_st", os.path.join(GOLDEN, "models", "Linear_16.onnx"), 1, "--safetensors", "--name", "Linear_16_st"))
    dynamic = []
    for m, make in DYNAMIC_MODELS.items():
        spec = make()
        p = os.path.join(OUT, m + ".onnx")
        ow.write(p, spec["nodes"], spec["inputs"], spec["outputs"], spec["init"], name=m)
        dynamic.append((m, p, len(spec["inputs"])))
    folded = reference_constant_folding_cases()
    multi = [("ElementwiseChains", elementwise_chains, 2), ("ParseRewrites", parse_rewrites, 3), ("ClassifierHead", classifier_head, 1),
             ("LayerNormBlock", layernorm_block, 1), ("ReduceBlock", reduce_block, 1), ("HardActivations", hard_activations, 2), ("IndexingBlock", indexing_block, 1)]
    multi += [(m, (lambda spec=spec: spec), len(spec["inputs"])) for m, spec in folded.items()]
    for m, spec in reference_stacked_matmul_cases().items():
        p = os.path.join(OUT, m + ".onnx")
        ow.write(p, spec["nodes"], spec["inputs"], spec["outputs"], spec["init"], name=m)
        emit_and_compile_dynamic(m, p, len(spec["inputs"]))
    for m, make, n_in in multi:
        spec = make()
        p = os.path.join(OUT, m + ".onnx")
        ow.write(p, spec["nodes"], spec["inputs"], spec["outputs"], spec["init"], name=m)
        _run([EMIT, p, OUT])
        src = os.path.join(OUT, m + "_harness.cxx")
        with open(src, "w") as f:
            f.write(MULTI_OUTPUT_HARNESS % dict(model=m, args=", ".join("inputs[%d]" % i for i in range(n_in))))
        compile_shared(src, os.path.join(OUT, "lib%s.so" % m))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda w: emit_and_compile(*w), work))
        list(ex.map(lambda w: emit_and_compile_dynamic(*w), dynamic))
    work += dynamic
    # models built through the RModel API (no ONNX file): sofie_hip_emit_example writes their headers
    _run([os.path.join(os.path.dirname(EMIT), "sofie_hip_emit_example"), OUT])
    for m in API_MODELS:
        compile_harness(m, 1)
    src = os.path.join(OUT, "ApiDynamicFp8Gemm_harness.cxx")
    with open(src, "w") as f:
        f.write(DYNAMIC_HARNESS % dict(model="ApiDynamicFp8Gemm", args="inputs[0]"))
    compile_shared(src, os.path.join(OUT, "libApiDynamicFp8Gemm.so"))
    compile_shared(os.path.join(ROOT, "tests", "harness_custom_memory.cxx"), os.path.join(OUT, "libCustomMemory.so"))
    compile_shared(os.path.join(ROOT, "tests", "harness_strided_input.cxx"), os.path.join(OUT, "libStridedInput.so"))
    return [w[0] for w in work] + list(API_MODELS) + ["ElementwiseChains", "ParseRewrites", "ClassifierHead", "LayerNormBlock", "ReduceBlock", "HardActivations", "IndexingBlock"]


if __name__ == "__main__":
    print("\n".join(build_all()))

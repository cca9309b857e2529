"""Sessions written by the C++ emitter, compiled at build time, run on the GPU and compared with the reference's
golden outputs and with the CPU oracle.  This is the user-visible path of the reference:
parse -> Generate -> OutputGenerated -> #include the header -> Session s(weights); s.infer(x)
(tests of the reference: core/test/TestCustomModelsFromONNX.cxx, the EmitFromONNX build step)."""
import ctypes
import os

import numpy as np
import pytest

from oracle import binding as ob
from sofie_amd import runtime as R
from tests import emitted_models as em
from tests import graph_runner as gr
from tests import onnx_lite
from tests.test_oracle_golden import MODELS, golden_tolerance

pytestmark = pytest.mark.gpu


def run_emitted(model, inputs, out_len):
    lib_path = os.path.join(em.OUT, "lib%s.so" % model)
    assert os.path.exists(lib_path), "emitted models are built by __graft_entry__.build()"
    lib = ctypes.CDLL(lib_path)
    err = ctypes.create_string_buffer(1024)
    arrs = [np.ascontiguousarray(a, dtype=np.float32) for a in inputs]
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    y = np.zeros(out_len, dtype=np.float32)
    rc = lib.run_model(os.path.join(em.OUT, model + "_GPU_HIP.dat").encode(), ptrs, y.ctypes.data_as(ctypes.c_void_p),
                       ctypes.c_ulong(out_len), err, 1024)
    assert rc == 0, err.value.decode()
    return y


@pytest.mark.parametrize("model", MODELS)
def test_emitted_session_reproduces_reference_golden_output(rt, model):
    g, inputs, expected = gr.load_fixture(model)
    print("emitted", model, flush=True)
    got = run_emitted(model, inputs, expected.size)
    assert np.abs(got - expected).max() <= golden_tolerance(model, expected)


def test_emitted_fp32_mlp_matches_oracle(rt):
    spec = em.fp32_mlp(64)
    g = onnx_lite.load(os.path.join(em.OUT, "Config1_fp32_MLP.onnx"))
    want = gr.run(g, spec["feeds"], gr.OracleBackend()).ravel()
    print("emitted Config1_fp32_MLP", flush=True)
    got = run_emitted("Config1_fp32_MLP", spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))


@pytest.mark.parametrize("model,dims,batch", [("Config2_int8_MLP_small", [64, 128, 96, 32], 48), ("Config2_int8_MLP_mid", [256, 512, 512, 256], 256)])
def test_emitted_int8_mlp_is_bit_exact(rt, model, dims, batch):
    from oracle import binding as ob
    spec = em.int8_mlp(dims, batch)
    c = spec["consts"]
    h = spec["feeds"][0]
    for l, w in enumerate(c["weights"]):   # the unfused ONNX chain, operator by operator
        q = ob.quantize_linear(h, c["in_scales"][l])
        acc = np.maximum(ob.matmul_integer(q, w, M=batch, N=w.shape[1], K=w.shape[0], omp=True), 0)
        h = ob.dequantize_linear(acc, np.float32(c["in_scales"][l] * c["w_scales"][l]))
    print("emitted", model, flush=True)
    got = run_emitted(model, spec["feeds"], h.size)
    assert np.array_equal(got.view(np.uint32), h.ravel().view(np.uint32))
    assert np.abs(h).max() > 0


def test_emitted_int8_mlp_at_full_size_on_sampled_rows(rt):
    """benchmark configuration 2 at its real size (1024 -> 4096 -> 4096 -> 1024, batch 1024) through the emitted Session that the
    benchmark times: weights from a safetensors file, input resident on the device, infer_nosync.  The rows of a batch are
    independent, so the unfused CPU chain runs on a sample of them: bit-exact."""
    from oracle import binding as ob
    spec = em.bench_mlp_spec()
    c, X = spec["consts"], spec["feeds"][0]
    rows = np.array([0, 1, 127, 128, 255, 256, 511, 777, 1022, 1023])
    h = np.ascontiguousarray(X[rows])
    for l, w in enumerate(c["weights"]):
        q = ob.quantize_linear(h, c["in_scales"][l])
        acc = np.maximum(ob.matmul_integer(q, w, M=len(rows), N=w.shape[1], K=w.shape[0], omp=True), 0)
        h = ob.dequantize_linear(acc, np.float32(c["in_scales"][l] * c["w_scales"][l]))
    print("emitted Config2_int8_MLP (full size)", flush=True)
    s = em.BenchSession()
    try:
        s.upload(X)
        s.run(1)
        got = s.download((1024, 1024))
        s.run(3)   # further inferences on the same Session give the same bits
        again = s.download((1024, 1024))
    finally:
        s.close()
    assert np.array_equal(got[rows].view(np.uint32), h.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    assert np.abs(h).max() > 0 and (got > 0).mean() > 0.1
    from sofie_amd.benchsupport import emitted as be
    txt = open(os.path.join(be.OUT, be.BENCH_MODEL + "_GPU_HIP.hxx")).read()
    assert txt.count("sofie_hip_gemm_i8(") == 3 and "SOFIE_I8OUT_I8_DQQ" in txt and "safetensors" in txt


def test_emitted_full_size_int8_cnn_sampled_images(rt):
    """benchmark configuration 5 at its full size (batch 256, 64 x 64 images) through the Session the generator emits, the one the
    benchmark times.  The images of a batch are independent, so the unfused CPU chain runs on a sample of them: the int8
    stages are bit-exact, the fp32 tail (average, Gemm) is held to 1e-5."""
    from oracle.chains import int8_cnn_oracle
    from sofie_amd.benchsupport import emitted as be
    spec = be.bench_cnn_spec()
    m, X = spec["consts"], spec["feeds"][0]
    sample = [0, 1, 85, 170, 254, 255]
    want = int8_cnn_oracle(m, np.ascontiguousarray(X[sample]))
    print("emitted Config5_int8_CNN (full size)", flush=True)
    s = be.BenchSession(be.CNN_MODEL)
    try:
        s.upload(X)
        s.run(1)
        got = s.download((256, 10))
        s.run(2)
        again = s.download((256, 10))
    finally:
        s.close()
    assert np.abs(got[sample] - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    txt = open(os.path.join(be.OUT, be.CNN_MODEL + "_GPU_HIP.hxx")).read()
    assert txt.count("sofie_hip_conv_i8(") == 4 and "planes summed for the GlobalAveragePool" in txt


def test_emitted_int8_gemm_8192_sampled_rows_and_columns(rt):
    """benchmark configuration 3 at M = N = K = 8192 as a one-operator model (QGemm + Relu parsed from ONNX, B re-laid out once
    in the constructor): the emitted Session's output on sampled full rows and columns, bit-exact against the oracle."""
    from oracle import binding as ob
    from sofie_amd.benchsupport import emitted as be
    spec = be.bench_gemm_spec()
    c, A = spec["consts"], spec["feeds"][0]
    n = 8192
    print("emitted Config3_int8_GEMM_8192", flush=True)
    s = be.BenchSession(be.GEMM_MODEL)
    try:
        s.upload(A)
        s.run(1)
        got = s.download((n, n), np.int8)
    finally:
        s.close()
    rows = np.array([0, 1, 255, 256, 4095, 4096, 8191, 777])
    want = ob.gemm_i8(np.ascontiguousarray(A[rows]), c["Bt"], M=len(rows), N=n, K=n, transB=1, omp=True, bias=c["bias"], scale=c["scale"],
                      relu_out=1, out=2)
    assert np.array_equal(got[rows], want)
    cols = np.array([0, 63, 64, 4097, 8191])
    want_c = ob.gemm_i8(A, np.ascontiguousarray(c["Bt"][cols]), M=n, N=len(cols), K=n, transB=1, omp=True, bias=c["bias"][cols],
                        scale=c["scale"][cols], relu_out=1, out=2)
    assert np.array_equal(got[:, cols], want_c)
    assert got.max() == 127 and (got == 0).mean() > 0.3


def test_emitted_int8_cnn_matches_cpu_chain(rt):
    """QuantizeLinear -> 4 x [QLinearConv + Relu] -> DequantizeLinear -> GlobalAveragePool -> Flatten -> Gemm, parsed from ONNX,
    emitted, compiled: the int8 stages are bit-exact by construction of the kernels (checked operator by operator in
    test_gpu_conv_i8), the fp32 tail is held to 1e-5."""
    from tests.refmodels import int8_cnn_oracle
    spec = em.int8_cnn(2, 12)
    want = int8_cnn_oracle(spec["consts"], spec["feeds"][0]).ravel()
    print("emitted Config5_int8_CNN_small", flush=True)
    got = run_emitted("Config5_int8_CNN_small", spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    assert np.abs(want).max() > 1e-3


def test_emitted_int8_cnn_whose_last_convolution_sums_its_planes(rt):
    """Planes of 256 pixels: the GlobalAveragePool joins the last QLinearConv, whose feature map is never stored."""
    from tests.refmodels import int8_cnn_oracle
    spec = em.int8_cnn(2, 16, (3, 64, 128))
    want = int8_cnn_oracle(spec["consts"], spec["feeds"][0]).ravel()
    print("emitted Int8_CNN_plane_sums", flush=True)
    got = run_emitted("Int8_CNN_plane_sums", spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    assert np.abs(want).max() > 1e-3
    txt = open(os.path.join(em.OUT, "Int8_CNN_plane_sums_GPU_HIP.hxx")).read()
    assert txt.count("SOFIE_I8OUT_I8_PLANE_SUMS") == 1 and "sofie_hip_plane_sums_take_average" in txt and "sofie_hip_global_avg_pool_i8" not in txt


def test_model_built_through_the_api_external_stream_option(rt):
    # Y = Relu(X[1,3] * ones[3,1] + 0.5): ones -> 3.5 (the reference's tests/alpaka/TestAlpakaExternalStream.cxx:34-37)
    got = run_emitted("ApiGemmRelu", [np.ones((1, 3), np.float32)], 1)
    assert got.tolist() == [3.5]
    got = run_emitted("ApiGemmRelu", [np.array([[-1.0, -2.0, 0.25]], np.float32)], 1)
    assert got.tolist() == [0.0]


def test_emitted_fp8_gemm_within_the_stated_bound(rt):
    from oracle import binding as ob
    from tests import util
    M, K, N = 48, 256, 96
    s, w8 = 2024, np.empty(N * K, dtype=np.uint8)
    for i in range(N * K):                      # the code sequence of sofie_amd/emit/tools/emit_example_api.cxx
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        w8[i] = (s >> 24) & 0xBE
    w8 = w8.reshape(N, K)
    bias = (0.25 * ((np.arange(N) % 7) - 3)).astype(np.float32)
    x = util.normal(77, M * K).reshape(M, K)
    xs, wsc = np.float32(0.03125), np.float32(0.0078125)
    a8 = ob.quantize_fp8(x, xs)
    want, abs_sum = ob.gemm_fp8(a8, w8, M=M, N=N, K=K, transB=1, bias=bias, scale=np.float32(xs * wsc), act=4, out=1, want_abs_sum=True)
    print("emitted ApiFp8Gemm", flush=True)
    got = run_emitted("ApiFp8Gemm", [x], M * N).reshape(M, N)
    bound = 1.2 * 2.0 ** -14 * abs_sum.astype(np.float64) * float(xs * wsc) + 1e-6
    assert np.all(np.abs(got.astype(np.float64) - want) <= bound)
    assert np.abs(want).max() > 0.5


def test_custom_memory_sessions(rt):
    """Options::kCustomMemory: the caller's MemoryProvider supplies the one block (tests/harness_custom_memory.cxx runs the
    scenarios of the reference's TestAlpakaCustomMemory.cxx and reports them line by line)."""
    lib = ctypes.CDLL(os.path.join(em.OUT, "libCustomMemory.so"))
    report = ctypes.create_string_buffer(8192)
    print("custom memory harness", flush=True)
    failures = lib.run_custom_memory(em.OUT.encode(), report, 8192)
    text = report.value.decode()
    print(text)
    assert failures == 0 and "FAIL" not in text and text.count("ok ") >= 14


def test_strided_input_sessions(rt):
    """Options::kStridedInput: the Session's constructor takes the strides of the graph inputs and the Gemm reads its operands
    through them: row padding as a row stride, column-major storage as the transposed operand (tests/harness_strided_input.cxx
    runs the Gemm scenarios of the reference's TestAlpakaStridedInput.cxx and reports them line by line)."""
    lib = ctypes.CDLL(os.path.join(em.OUT, "libStridedInput.so"))
    report = ctypes.create_string_buffer(8192)
    print("strided input sessions", flush=True)
    failures = lib.run_strided_input(em.OUT.encode(), report, 8192)
    text = report.value.decode()
    assert failures == 0 and "FAIL" not in text and text.count("ok ") >= 26, text


def test_emitted_conv_batchnorm_relu(rt):
    spec = em.conv_batchnorm_relu(2)
    g = onnx_lite.load(os.path.join(em.OUT, "ConvBatchNormRelu.onnx"))
    want = gr.run(g, spec["feeds"], gr.OracleBackend()).ravel()
    print("emitted ConvBatchNormRelu", flush=True)
    got = run_emitted("ConvBatchNormRelu", spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    txt = open(os.path.join(em.OUT, "ConvBatchNormRelu_GPU_HIP.hxx")).read()
    assert "BatchNorm + ReLU" in txt and "sofie_hip_unary_f32" not in txt   # the Relu is folded into the normalisation


def test_emitted_conv_pool_stack(rt):
    spec = em.conv_pool_stack(2)
    g = onnx_lite.load(os.path.join(em.OUT, "ConvPoolStack.onnx"))
    want = gr.run(g, spec["feeds"], gr.OracleBackend()).ravel()
    print("emitted ConvPoolStack", flush=True)
    got = run_emitted("ConvPoolStack", spec["feeds"], want.size)
    assert want.size == 10 and np.abs(want).max() > 1e-2
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
    txt = open(os.path.join(em.OUT, "ConvPoolStack_GPU_HIP.hxx")).read()
    # 10x10 -> MaxPool(3, stride 2, pad 1) -> 5x5 -> AveragePool(2, stride 2, ceil) -> 3x3, its divisor following the window
    assert "d.OH = 5; d.OW = 5;" in txt and "d.OH = 3; d.OW = 3;" in txt and "d.dynamic_divisor = 1" in txt


def test_safetensors_session_reproduces_the_golden_output(rt, tmp_path):
    from safetensors.numpy import load_file, save_file
    g, inputs, expected = gr.load_fixture("Linear_16")
    lib = ctypes.CDLL(os.path.join(em.OUT, "libLinear_16_st.so"))
    x = np.ascontiguousarray(inputs[0], dtype=np.float32)
    ptrs = (ctypes.c_void_p * 1)(x.ctypes.data)
    # the file the generator wrote, and the same tensors re-saved by the safetensors library (with metadata)
    own = os.path.join(em.OUT, "Linear_16_st_GPU_HIP.safetensors")
    resaved = str(tmp_path / "resaved.safetensors")
    save_file(dict(reversed(list(load_file(own).items()))), resaved, metadata={"producer": "test"})
    for path in (own, resaved):
        y = np.zeros(expected.size, dtype=np.float32)
        err = ctypes.create_string_buffer(1024)
        print("safetensors", path, flush=True)
        rc = lib.run_model(path.encode(), ptrs, y.ctypes.data_as(ctypes.c_void_p), ctypes.c_ulong(y.size), err, 1024)
        assert rc == 0, err.value.decode()
        assert np.abs(y - expected).max() <= golden_tolerance("Linear_16", expected)


def test_emitted_qlinear_matmul_relu_is_bit_exact(rt):
    from oracle import binding as ob
    spec = em.qlinear_matmul_relu()
    c, x = spec["consts"], spec["feeds"][0]
    M, K = x.shape
    N = c["W"].shape[1]
    q = ob.quantize_linear(x, c["sx"])
    y8 = ob.gemm_i8(q, c["W"], M=M, N=N, K=K, scale=c["mult"], relu_out=1, out=2)
    want = ob.dequantize_linear(y8, c["sy"])
    print("emitted QLinearMatMulRelu", flush=True)
    got = run_emitted("QLinearMatMulRelu", [x], M * N).reshape(M, N)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert (y8 > 0).any() and (y8 == 0).any()
    txt = open(os.path.join(em.OUT, "QLinearMatMulRelu_GPU_HIP.hxx")).read()
    assert "d.relu_out = 1" in txt and "SOFIE_I8OUT_I8;" in txt and "sofie_hip_unary_f32" not in txt


def test_emitted_conv_integer_chain_is_bit_exact(rt):
    from oracle import binding as ob
    spec = em.conv_integer_dequantize()
    c, x = spec["consts"], spec["feeds"][0]
    q = ob.quantize_linear(x, c["sx"])
    acc = ob.conv_i8(q, c["W"], None, None, pads=(1, 1, 1, 1), relu=1, out=0)
    want = ob.dequantize_linear(acc, c["sacc"])
    print("emitted ConvIntegerDequantize", flush=True)
    got = run_emitted("ConvIntegerDequantize", [x], want.size).reshape(want.shape)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert (acc > 0).any()


VIEW_MODELS = [("Linear_16", None), ("ConvWithPadding", None), ("LinearWithSigmoid", None), ("Config1_fp32_MLP", lambda: em.fp32_mlp(64)),
               ("Config2_int8_MLP_small", lambda: em.int8_mlp([64, 128, 96, 32], 48)), ("Config5_int8_CNN_small", lambda: em.int8_cnn(2, 12)),
               ("ConvBatchNormRelu", lambda: em.conv_batchnorm_relu(2))]


@pytest.mark.parametrize("misalign", [0, 3])
@pytest.mark.parametrize("model,make", VIEW_MODELS)
def test_infer_on_views_of_device_memory_equals_infer_on_host_pointers(rt, model, make, misalign):
    """infer(std::span<ViewConstF1D const>, std::span<ViewF1D>) (the reference's third infer signature): in place on
    aligned views, through the session's regions otherwise; either way the bits of infer(host pointers)."""
    if make:
        spec = make()
        inputs, out_len = spec["feeds"], int(np.prod(spec["outputs"][0][2]))
    else:
        _, inputs, expected = gr.load_fixture(model)
        out_len = int(expected.size)
    arrs = [np.ascontiguousarray(a, dtype=np.float32) for a in inputs]
    lib = ctypes.CDLL(os.path.join(em.OUT, "lib%s.so" % model))
    err = ctypes.create_string_buffer(1024)
    weights = os.path.join(em.OUT, model + "_GPU_HIP.dat").encode()
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    lens = (ctypes.c_ulong * len(arrs))(*[a.size for a in arrs])
    want = run_emitted(model, arrs, out_len)
    got = np.zeros(out_len, dtype=np.float32)
    print("views", model, "misalign", misalign, flush=True)
    rc = lib.run_model_views(weights, ptrs, lens, len(arrs), got.ctypes.data_as(ctypes.c_void_p), ctypes.c_ulong(out_len), misalign, err, 1024)
    assert rc == 0, err.value.decode()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)) and np.abs(want).max() > 0


def test_emitted_elementwise_chains(rt):
    """One-to-one operators folded behind a Gemm, behind a Conv and behind one another (the reference's elementwise fusion,
    core/inc/SOFIE/operators/ROperator_ALPAKA.hxx:57-76), against the same operators run one by one on the CPU."""
    spec = em.elementwise_chains()
    g = onnx_lite.load(os.path.join(em.OUT, "ElementwiseChains.onnx"))
    want = np.concatenate([w.ravel() for w in gr.run(g, spec["feeds"], gr.OracleBackend(), all_outputs=True)])
    print("emitted ElementwiseChains", flush=True)
    got = run_emitted("ElementwiseChains", spec["feeds"], want.size)
    assert np.all(np.abs(got - want) <= 1e-5 * np.maximum(1.0, np.abs(want)))
    txt = open(os.path.join(em.OUT, "ElementwiseChains_GPU_HIP.hxx")).read()
    body = txt[txt.index("void doInfer("):txt.index("void infer_nosync(")]
    # 18 operators in the graph, 5 launches
    assert body.count("detail::Check(") == 5 and body.count("sofie_hip_unary_chain_f32") == 2 and body.count("sofie_hip_unary_f32") == 1


def test_emitted_classifier_head_with_softmax_and_logsoftmax(rt):
    spec = em.classifier_head(4)
    g = onnx_lite.load(os.path.join(em.OUT, "ClassifierHead.onnx"))
    P, Q = gr.run(g, spec["feeds"], gr.OracleBackend(), all_outputs=True)
    print("emitted ClassifierHead", flush=True)
    got = run_emitted("ClassifierHead", spec["feeds"], P.size + Q.size)
    gp, gq = got[:P.size].reshape(P.shape), got[P.size:].reshape(Q.shape)
    assert np.all(np.abs(gp - P) <= 1e-5 * P + 1e-7) and np.allclose(gp.sum(axis=1), 1.0, atol=1e-5)
    assert np.all(np.abs(gq - Q) <= 1e-5 * np.abs(Q) + 1e-5) and P.std() > 0.01
    txt = open(os.path.join(em.OUT, "ClassifierHead_GPU_HIP.hxx")).read()
    assert txt.count("sofie_hip_softmax_f32(") == 2 and "sofie_hip_gemm_chain_f32(fCtx, chain, 2)" in txt


def test_emitted_gemm_chain_of_different_widths(rt):
    """Three Gemms of widths 128 / 64 / 96 emitted as one chain call, then Softmax: the Session's own memory plan under the
    one-launch kernel."""
    spec = em.gemm_chain_widths(64)
    g = onnx_lite.load(os.path.join(em.OUT, "GemmChainWidths.onnx"))
    want = gr.run(g, spec["feeds"], gr.OracleBackend()).ravel()
    print("emitted GemmChainWidths", flush=True)
    got = run_emitted("GemmChainWidths", spec["feeds"], want.size)
    assert np.all(np.abs(got - want) <= 1e-5 * want + 1e-7) and want.std() > 1e-4


def test_emitted_layernorm_block(rt):
    spec = em.layernorm_block(3)
    X = spec["feeds"][0]
    i = spec["init"]
    H = ob.gemm_f32(X, i["W1"], i["b1"], M=3, N=16, K=12, bias_mode=1)
    N, mean, _ = ob.layernorm(H, i["g"], i["beta"], -1, 1e-5, stats=True)
    Y = ob.gemm_f32(ob.unary(N, R.ACT_GELU), i["W2"], None, M=3, N=4, K=16)
    print("emitted LayerNormBlock", flush=True)
    got = run_emitted("LayerNormBlock", spec["feeds"], 12 + 3)
    assert np.abs(got[:12] - Y.ravel()).max() <= 3e-5 * max(1.0, float(np.abs(Y).max())) and np.allclose(got[12:], mean, rtol=1e-5, atol=1e-6)
    assert Y.std() > 0.05


def test_emitted_hard_activations_ride_in_the_stores(rt):
    spec = em.hard_activations(4)
    g = onnx_lite.load(os.path.join(em.OUT, "HardActivations.onnx"))
    Y, V = gr.run(g, spec["feeds"], gr.OracleBackend(), all_outputs=True)
    print("emitted HardActivations", flush=True)
    got = run_emitted("HardActivations", spec["feeds"], Y.size + V.size)
    gy, gv = got[:Y.size].reshape(Y.shape), got[Y.size:].reshape(V.shape)
    assert np.abs(gy - Y).max() <= 1e-5 and np.abs(gv - V).max() <= 1e-5 * max(1.0, float(np.abs(V).max()))
    assert 0.0 <= Y.min() and Y.max() <= 1.0 and Y.std() > 0.05 and (V == 0).any() and V.max() > 3.0       # both clamps of HardSwish are reached
    txt = open(os.path.join(em.OUT, "HardActivations_GPU_HIP.hxx")).read()
    assert "sofie_hip_unary" not in txt and txt.count("SOFIE_ACT_HARDSWISH") == 2 and "SOFIE_ACT_SWISH" in txt and "SOFIE_ACT_HARDSIGMOID" in txt


def indexing_block_expected(X):
    """numpy's own indexing, output after output"""
    A, B, Cc = X[:, :, 0:3], X[:, :, 3:6], X[:, :, 6:8]
    S = X[:, ::-2, 1:7]
    G = X[:, [4, -1, 0], :]
    T = np.tile(Cc, (1, 2, 3))
    E = np.broadcast_to(X[:, [2], :], (X.shape[0], 5, 8))
    return np.concatenate([np.ascontiguousarray(v, dtype=np.float32).ravel() for v in (A + B, S, G, T, E)])


def test_emitted_indexing_block(rt):
    spec = em.indexing_block(3)
    want = indexing_block_expected(spec["feeds"][0])
    print("emitted IndexingBlock", flush=True)
    got = run_emitted("IndexingBlock", spec["feeds"], want.size)
    assert want.size == 3 * (18 + 18 + 24 + 72 + 40) and np.array_equal(got, want)
    g = onnx_lite.load(os.path.join(em.OUT, "IndexingBlock.onnx"))
    outs = gr.run(g, spec["feeds"], gr.OracleBackend(), all_outputs=True)      # the graph runner's reading of the same operators agrees
    assert np.array_equal(np.concatenate([o.ravel() for o in outs]), want)


def test_emitted_reduce_block(rt):
    spec = em.reduce_block(3)
    X = spec["feeds"][0]
    C = ob.binary_broadcast(X, ob.reduce(X, R.REDUCE_MEAN, [2], 1), 1)
    want = np.concatenate([ob.reduce(C, R.REDUCE_L2, [-1], 0).ravel(), ob.reduce(X, R.REDUCE_MAX, [1], 0).ravel(), ob.reduce(X, R.REDUCE_SUM, [0], 1).ravel()])
    print("emitted ReduceBlock", flush=True)
    got = run_emitted("ReduceBlock", spec["feeds"], want.size)
    assert want.size == 12 + 18 + 24 and np.array_equal(got, want) and want.std() > 0.3
    # float64 numpy as a second opinion on the whole graph
    x64 = X.astype(np.float64)
    ref = np.concatenate([np.sqrt(((x64 - x64.mean(axis=2, keepdims=True)) ** 2).sum(axis=2)).ravel(), x64.max(axis=1).ravel(), x64.sum(axis=0).ravel()])
    assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()


def test_emitted_shape_plumbing(rt):
    spec = em.shape_plumbing(3)
    g = onnx_lite.load(os.path.join(em.OUT, "ShapePlumbing.onnx"))
    want = gr.run(g, spec["feeds"], gr.OracleBackend()).ravel()
    print("emitted ShapePlumbing", flush=True)
    got = run_emitted("ShapePlumbing", spec["feeds"], want.size)
    assert want.size == 18 and np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max())) and want.std() > 0.05


def test_emitted_residual_block(rt):
    """Adds of equal-shaped tensors behind a Conv and a Gemm ride in those operators' stores (tests/emitted_models.residual_block)."""
    spec = em.residual_block(2)
    g = onnx_lite.load(os.path.join(em.OUT, "ResidualBlock.onnx"))
    want = gr.run(g, spec["feeds"], gr.OracleBackend()).ravel()
    print("emitted ResidualBlock", flush=True)
    got = run_emitted("ResidualBlock", spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-5 and want.std() > 0.01


def test_emitted_parse_time_rewrites(rt):
    """Cast to the same type, Transpose -> MatMul, MatMul + Add, Conv + Add(1-D initializer), a Gemm of weights only:
    the rewrites of the reference's parser and the fold of its Gemm, against the definitions in float64."""
    spec = em.parse_rewrites()
    want = np.concatenate([w.ravel() for w in spec["want"]])
    print("emitted ParseRewrites", flush=True)
    got = run_emitted("ParseRewrites", spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))


@pytest.mark.parametrize("model", ["Gemm_ConstantFolding", "Gemm_ConstantFolding_Shared", "MatMul_1D_Constant"])
def test_constant_folding_cases_of_the_reference(rt, model):
    """The reference's own tests with their literal expectations (tests/cpu/TestCustomModelsFromONNX.cxx:509-527, 1672-1677):
    products of weights are folded when the code is generated, a Session without inputs still answers."""
    spec = em.reference_constant_folding_cases()[model]
    want = np.concatenate([np.asarray(w, np.float32) for w in spec["want"]])
    print("emitted", model, flush=True)
    got = run_emitted(model, spec["feeds"], want.size)
    assert np.abs(got - want).max() <= 1e-3                 # DEFAULT_TOLERANCE of the reference's tests
    assert np.array_equal(got, want)                        # small integers: exact in fp32 in any order
    txt = open(os.path.join(em.OUT, model + "_GPU_HIP.hxx")).read()
    assert "computed when the code was generated" in txt

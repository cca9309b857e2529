"""The C++ emitter (sofie_amd/emit): the text it generates and its memory plan, checked on the CPU.
Reference behaviour mirrored: RModel::GenerateSessionCode (core/src/RModel.cxx:1167-1460), the planner
OrganizeMemory (core/inc/SOFIE/MemoryPlanner.inc:67-170) and the Session/infer API of the generated code."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from tests import emitted_models as em
from tests import onnx_write as ow


@pytest.fixture(scope="module")
def emitted():
    if not os.path.exists(os.path.join(em.OUT, "libLinear_16.so")):
        em.build_all()
    return em.OUT


def ops_body(txt):
    """The statements of the operators: the body of Session::doInfer."""
    body = txt[txt.index("void doInfer("):]
    return body[:body.index("void infer_nosync(")]


def plan_of(onnx_path, tmp_path):
    out = subprocess.run([em.EMIT, onnx_path, str(tmp_path), "--plan"], check=True, stdout=subprocess.PIPE, text=True).stdout.split("\n")
    head = out[0].split()
    rows = []
    for line in out[1:]:
        f = line.split()
        if len(f) == 6:
            rows.append(dict(name=f[0], offset=int(f[1]), bytes=int(f[2]), first=int(f[3]), last=int(f[4]), pooled=int(f[5])))
    return int(head[1]), int(head[3]), rows


def test_linear16_pool_matches_the_reference_planner(emitted, tmp_path):
    # the reference's GPU planner gives 6656 bytes for this model (two 3200-byte activations alive at once,
    # each rounded to 256): same figure from oracle/_ref's build of MemoryPlanner.inc in test_oracle_pins
    arena, pool, rows = plan_of(os.path.join(em.GOLDEN, "models", "Linear_16.onnx"), tmp_path)
    assert pool == 6656
    assert arena == max(r["offset"] + r["bytes"] for r in rows)


@pytest.mark.parametrize("model", ["Linear_16", "ConvWithPadding", "LinearWithSigmoid", "Config1_fp32_MLP", "Config2_int8_MLP_mid"])
def test_plan_alignment_and_liveness(emitted, tmp_path, model):
    path = os.path.join(em.GOLDEN, "models", model + ".onnx")
    if not os.path.exists(path):
        path = os.path.join(emitted, model + ".onnx")
    arena, pool, rows = plan_of(path, tmp_path)
    assert rows
    for r in rows:
        assert r["offset"] % 256 == 0 and r["offset"] + r["bytes"] <= arena
    for i, a in enumerate(rows):
        for b in rows[i + 1:]:
            overlap_mem = a["offset"] < b["offset"] + b["bytes"] and b["offset"] < a["offset"] + a["bytes"]
            if not overlap_mem:
                continue
            if 2 in (a["pooled"], b["pooled"]) and a["offset"] == b["offset"] and a["bytes"] == b["bytes"]:
                continue    # a view (Reshape, Flatten ...) lies on the tensor it is a view of
            # sharing bytes is allowed only between pooled tensors whose lifetimes are disjoint
            assert a["pooled"] and b["pooled"], (a, b)
            assert a["last"] <= b["first"] or b["last"] <= a["first"], (a, b)
    pooled = [r for r in rows if r["pooled"]]
    if pooled:
        lo = min(r["offset"] for r in pooled)
        assert max(r["offset"] + r["bytes"] for r in pooled) - lo == pool
        assert pool <= sum(r["bytes"] for r in pooled)


def test_tensors_of_a_gemm_chain_share_no_memory(emitted, tmp_path):
    """Three Gemms of different widths that go to the runtime as one call (which may run them in one launch, every workgroup
    taking its rows through all the layers): tensors of different shape would share memory under per-operator lifetimes, so
    the chain's input, outputs and biases are planned as live for the whole chain.  (Equal shapes may share row for row: the
    reference's ping-pong of Linear_16 stays, see test_linear16_pool_matches_the_reference_planner.)"""
    arena, pool, rows = plan_of(os.path.join(emitted, "GemmChainWidths.onnx"), tmp_path)
    txt = read(emitted, "GemmChainWidths")
    assert "sofie_hip_gemm_chain_f32(fCtx, chain, 3)" in txt
    chain = [r for r in rows if r["name"] in ("tensor_X", "tensor_Y0", "tensor_Y1", "tensor_Y2", "tensor_b0", "tensor_b1", "tensor_b2",
                                              "tensor_W0", "tensor_W1", "tensor_W2")]
    assert len(chain) == 10
    for i, a in enumerate(chain):
        for b in chain[i + 1:]:
            assert a["offset"] + a["bytes"] <= b["offset"] or b["offset"] + b["bytes"] <= a["offset"], (a, b)
    y = {r["name"]: r for r in rows}
    assert y["tensor_Y0"]["first"] == 0 and y["tensor_Y0"]["last"] >= 3 and y["tensor_Y1"]["first"] == 0 and y["tensor_Y2"]["first"] == 0


def read(emitted, model):
    return open(os.path.join(emitted, model + "_GPU_HIP.hxx")).read()


def test_session_api_of_the_generated_header(emitted):
    txt = read(emitted, "Linear_16")
    assert "namespace SOFIE_Linear_16" in txt and "struct Session" in txt
    assert re.search(r'Session\(std::string filename = "Linear_16_GPU_HIP\.dat"', txt)
    assert re.search(r"std::vector<float> infer\(float const ?\*", txt)
    assert "void infer_nosync()" in txt
    assert "#include \"sofie_hip.h\"" in txt
    # nothing in the generated code may allocate per inference
    body = txt[txt.index("void doInfer("):]
    body = body[:body.index("std::vector<float> infer(")]
    assert "arena_create" not in body and "hipMalloc" not in body and "new " not in body


def test_gemm_relu_pairs_are_fused(emitted):
    txt = read(emitted, "Linear_16")
    body = ops_body(txt)
    # ten layers, each reading its predecessor: one chain call
    assert body.count("sofie_hip_gemm_chain_f32(fCtx, chain, 10)") == 1 and "sofie_hip_gemm_f32(" not in body
    assert "sofie_hip_unary_f32" not in body          # every Relu went into a Gemm epilogue
    assert body.count(".act = SOFIE_ACT_RELU") == 9
    txt = read(emitted, "LinearWithSigmoid")
    assert "SOFIE_ACT_SIGMOID" in txt


def test_quantised_chain_collapses_to_one_kernel_per_layer(emitted):
    txt = read(emitted, "Config2_int8_MLP_mid")
    body = ops_body(txt)
    assert body.count("sofie_hip_gemm_i8(") == 3
    assert body.count("sofie_hip_quantize_linear(") == 1    # only the model input is quantised by its own kernel
    assert "sofie_hip_dequantize_linear" not in body        # the last DequantizeLinear is the GEMM's fp32 store
    assert body.count("SOFIE_I8OUT_I8_DQQ") == 2 and body.count("SOFIE_I8OUT_F32") == 1


def test_conv_is_emitted_as_one_call_with_resolved_geometry(emitted):
    txt = read(emitted, "ConvWithAsymmetricPadding")
    assert txt.count("sofie_hip_conv_f32(") == 1
    assert "im2col" not in txt.lower().replace("implicit im2col", "")


def _emit(tmp_path, nodes, inputs, outputs, init, name="m"):
    p = os.path.join(str(tmp_path), name + ".onnx")
    ow.write(p, nodes, inputs, outputs, init, name=name)
    return subprocess.run([em.EMIT, p, str(tmp_path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_reshapes_of_pool_tensors_are_views(tmp_path):
    """Operators that hand their input's bytes on unchanged generate no copy when input and output both live in the pool: the
    output is placed on the input, and the tensor at the root of a chain of views lives until the last reader of any of them.
    A graph input or output has a region of its own, so a Reshape that reads or writes one still copies."""
    init = {"shape": np.array([4, 6], dtype=np.int64), "shape2": np.array([6, 4], dtype=np.int64)}
    nodes = [ow.node("Reshape", ["X", "shape2"], ["X2"]),    # 0: reads a graph input: a copy
             ow.node("Relu", ["X2"], ["A"]),                 # 1
             ow.node("Flatten", ["A"], ["F"], axis=0),       # 2: a view of A ([1, 24])
             ow.node("Reshape", ["F", "shape"], ["G"]),      # 3: a view of a view
             ow.node("Exp", ["G"], ["Y"]),                   # 4
             ow.node("Neg", ["A"], ["N"]),                   # 5: A is read again behind the views
             ow.node("Reshape", ["N", "shape"], ["Z"])]      # 6: writes a graph output: a copy
    p = os.path.join(str(tmp_path), "views.onnx")
    ow.write(p, nodes, [("X", np.float32, [2, 3, 4])], [("Y", np.float32, [4, 6]), ("Z", np.float32, [4, 6])], init, name="views")
    out = subprocess.run([em.EMIT, p, str(tmp_path), "--plan"], check=True, stdout=subprocess.PIPE, text=True).stdout.split("\n")
    rows = {f[0]: dict(offset=int(f[1]), bytes=int(f[2]), first=int(f[3]), last=int(f[4]), kind=int(f[5])) for f in (l.split() for l in out[1:]) if len(f) == 6}
    assert rows["tensor_F"]["kind"] == 2 and rows["tensor_G"]["kind"] == 2 and rows["tensor_A"]["kind"] == 1 and rows["tensor_X2"]["kind"] == 1
    assert rows["tensor_F"]["offset"] == rows["tensor_G"]["offset"] == rows["tensor_A"]["offset"]
    assert rows["tensor_A"]["first"] == 1 and rows["tensor_A"]["last"] == 6      # through Neg (operator 5), past Exp (4), the views' reader
    # nothing else may take A's bytes while its views are read
    for n, r in rows.items():
        if r["kind"] == 1 and n != "tensor_A" and r["offset"] < rows["tensor_A"]["offset"] + rows["tensor_A"]["bytes"] and \
           rows["tensor_A"]["offset"] < r["offset"] + r["bytes"]:
            assert r["last"] <= 1 or r["first"] >= 6, (n, r)
    body = ops_body(open(os.path.join(str(tmp_path), "views_GPU_HIP.hxx")).read())
    assert "tensor_F is a view of tensor_A" in body and "tensor_G is a view of tensor_F" in body
    assert body.count("sofie_hip_copy(") == 2 and "sofie_hip_copy(fCtx, tensor_X2, tensor_X" in body and "sofie_hip_copy(fCtx, tensor_Z, tensor_N" in body
    assert "SOFIE_ACT_EXP" in body and "tensor_G" in body[body.index("SOFIE_ACT_EXP") - 200:body.index("SOFIE_ACT_EXP") + 200]


def test_strided_input_option_adds_the_strides_to_the_session(emitted):
    """Options::kStridedInput (core/src/RModel.cxx:1272-1300, 1546-1549 of the reference): the constructor takes one stride array
    per input behind the shape parameter, checks count and rank with the reference's messages, and the Gemm resolves the row
    stride and the transpose flag of a strided operand when it runs."""
    txt = read(emitted, "StridedGemmAB")
    assert 'Session(std::string filename = "", std::vector<std::vector<std::size_t>> inputStrides = {}, int device = 0)' in txt
    assert "std::vector<std::size_t> fInputStride_A;" in txt and "std::vector<std::size_t> fInputStride_B;" in txt
    assert "sofie: expected 2 input stride array(s), one per input tensor" in txt
    assert "sofie: the stride array of input tensor B must have 2 element(s)" in txt
    body = ops_body(txt)
    assert "d.transA = !d.transA;" in body and "d.ldb = static_cast<std::int32_t>(std::max<std::size_t>(this->fInputStride_B[0]" in body
    assert "without a unit stride, which BLAS cannot handle" in body
    # the arena grows by the extents of the inputs that came with strides, and those inputs live there
    assert "sofie_hip_arena_create(fCtx, kArenaBytes + sofie_strided_bytes, 256)" in txt
    assert "tensor_A = reinterpret_cast<float *>(base + kArenaBytes + sofie_strided_offset_A);" in txt
    # the shape parameter comes first, as in the reference's signature
    dyn = read(emitted, "StridedGemmDynamic")
    assert 'std::size_t N = 8, std::vector<std::vector<std::size_t>> inputStrides = {}, int device = 0)' in dyn
    assert "InputExtent_X(fMaxBatch)" in dyn and "InputExtent_X(N) * 4" in dyn
    # without the option nothing of it is emitted
    assert "inputStrides" not in read(emitted, "ApiGemmRelu")


def _emit_strided(tmp_path, nodes, inputs, outputs, init, name="m"):
    p = os.path.join(str(tmp_path), name + ".onnx")
    ow.write(p, nodes, inputs, outputs, init, name=name)
    return subprocess.run([em.EMIT, p, str(tmp_path), "--strided-input"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def test_strided_input_is_refused_where_no_operator_can_read_it(tmp_path):
    """The refusals of the reference at generation (tests/cpu/TestStridedInput.cxx:198-208, 261-274; ROperator_Gemm.hxx:394-399):
    an operator that cannot read through strides, a strided bias, a strided operand that is not a plain 2-D matrix."""
    W = {"W": np.zeros((4, 3), dtype=np.float32)}
    r = _emit_strided(tmp_path, [ow.node("Relu", ["X"], ["Y"])], [("X", np.float32, [2, 4])], [("Y", np.float32, [2, 4])], {})
    assert r.returncode != 0 and "Options::kStridedInput" in r.stdout and "reads the input tensor X but does not support strided input access" in r.stdout
    r = _emit_strided(tmp_path, [ow.node("Gemm", ["X", "W", "C"], ["Y"])], [("X", np.float32, [2, 4]), ("C", np.float32, [2, 3])],
                      [("Y", np.float32, [2, 3])], W)
    assert r.returncode != 0 and "strided input is not supported for the bias (C)" in r.stdout
    r = _emit_strided(tmp_path, [ow.node("MatMul", ["X", "W"], ["Y"])], [("X", np.float32, [5, 2, 4])], [("Y", np.float32, [5, 2, 3])], W)
    assert r.returncode != 0 and "strided input is only supported for a plain 2D Gemm" in r.stdout
    # the same Gemm with only its A operand a graph input is taken, and an activation behind it still joins its store
    r = _emit_strided(tmp_path, [ow.node("Gemm", ["X", "W"], ["H"]), ow.node("Relu", ["H"], ["Y"])], [("X", np.float32, [2, 4])],
                      [("Y", np.float32, [2, 3])], W, name="ok")
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), "ok_GPU_HIP.hxx")).read()
    assert "fInputStride_X" in ops_body(txt) and "SOFIE_ACT_RELU" in ops_body(txt)


def test_unsupported_operator_is_refused_by_name(tmp_path):
    r = _emit(tmp_path, [ow.node("LSTM", ["X"], ["Y"])], [("X", np.float32, [1, 4])], [("Y", np.float32, [1, 4])], {})
    assert r.returncode != 0 and "LSTM" in r.stdout


def test_shape_mismatch_is_refused(tmp_path):
    init = {"W": np.zeros((5, 3), dtype=np.float32)}
    r = _emit(tmp_path, [ow.node("Gemm", ["X", "W"], ["Y"])], [("X", np.float32, [2, 4])], [("Y", np.float32, [2, 3])], init)
    assert r.returncode != 0 and "Gemm" in r.stdout


def test_missing_input_tensor_is_refused(tmp_path):
    r = _emit(tmp_path, [ow.node("Relu", ["nope"], ["Y"])], [("X", np.float32, [2, 4])], [("Y", np.float32, [2, 4])], {})
    assert r.returncode != 0 and "nope" in r.stdout


def test_session_fails_loudly_without_a_gpu(emitted):
    import torch
    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU")
    lib = ctypes.CDLL(os.path.join(emitted, "libLinear_16.so"))
    err = ctypes.create_string_buffer(512)
    x = np.ones(1600, dtype=np.float32)
    y = np.zeros(160, dtype=np.float32)
    inp = (ctypes.c_void_p * 1)(x.ctypes.data)
    rc = lib.run_model(os.path.join(emitted, "Linear_16_GPU_HIP.dat").encode(), inp, y.ctypes.data_as(ctypes.c_void_p), ctypes.c_ulong(160), err, 512)
    assert rc == 1 and b"SOFIE HIP runtime error" in err.value
    assert not y.any()


def test_weight_file_round_trip(emitted):
    # the .dat file holds every initialised tensor as "name count" + values, fp32 printed so that it reads back exactly
    from tests import onnx_lite
    g = onnx_lite.load(os.path.join(em.GOLDEN, "models", "Linear_16.onnx"))
    toks = open(os.path.join(emitted, "Linear_16_GPU_HIP.dat")).read().split()
    i, seen = 0, {}
    while i < len(toks):
        name, n = toks[i], int(toks[i + 1])
        seen[name] = np.array([float(t) for t in toks[i + 2:i + 2 + n]], dtype=np.float32)
        i += 2 + n
    assert len(seen) == len(g["initializers"])
    for k, v in g["initializers"].items():
        key = "tensor_" + re.sub(r"[^A-Za-z0-9_]", "_", k)
        assert np.array_equal(seen[key], np.asarray(v, dtype=np.float32).ravel()), k


def test_quantised_cnn_keeps_channels_last_and_reads_activations_in_place(emitted):
    txt = read(emitted, "Config5_int8_CNN_small")
    body = ops_body(txt)
    assert body.count("sofie_hip_conv_i8(") == 4
    assert "sofie_hip_unary_f32" not in body                      # the four Relu are in the convolutions' stores
    assert body.count("a.relu = 1") == 4
    # no column matrix anywhere: the 3-channel input's rows (K = 27) are gathered inside the kernel
    assert body.count("implicit GEMM") == 3 and body.count("rows gathered in the kernel") == 1 and "workspace" not in body
    assert body.count("a.y_layout = SOFIE_LAYOUT_NHWC") == 4
    assert body.count("a.x_layout = SOFIE_LAYOUT_NCHW") == 1     # the quantised model input
    assert "sofie_hip_dequantize_linear" not in body and "sofie_hip_global_avg_pool_i8(" in body
    # weights are re-laid out once, in the constructor
    ctor = txt[txt.index("Session(std::string filename"):txt.index("void doInfer(")]
    assert ctor.count("sofie_hip_pack_conv_weight_i8(") == 4


def test_global_average_pool_joins_a_convolution_whose_planes_the_runtime_can_sum(emitted):
    txt = read(emitted, "Int8_CNN_plane_sums")
    body = ops_body(txt)
    assert body.count("sofie_hip_conv_i8(") == 2 and body.count("a.out = SOFIE_I8OUT_I8_PLANE_SUMS") == 1
    assert "sofie_hip_global_avg_pool_i8(" not in body and body.count("sofie_hip_plane_sums_take_average(") == 1
    # a buffer of the operator's own (2 images x 128 channels of int32), cleared once in the constructor; every inference sums
    # into it and the averaging call clears it again behind its read: no clearing launch per inference
    assert "sofie_hip_fill_zero(" not in body and "workspace_op_2" not in body
    ctor = txt[txt.index("Session(std::string filename"):txt.index("void doInfer(")]
    assert ctor.count("sofie_hip_fill_zero(fCtx, planesums_") == 1 and ", 1024), " in ctor[ctor.index("sofie_hip_fill_zero(fCtx, planesums_"):][:200]
    order = [body.index(k) for k in ("a.Y = planesums_", "sofie_hip_conv_i8(fCtx, &d, &a), \"op_2", "sofie_hip_plane_sums_take_average(fCtx, tensor_")]
    assert order[0] < order[1] < order[2]
    assert ", 256, 256, " in body[order[2]:order[2] + 300]        # 256 sums, planes of 256 pixels
    # planes of 144 pixels (12 x 12) stay with the stand-alone kernel
    assert "PLANE_SUMS" not in read(emitted, "Config5_int8_CNN_small")
    # with a run-time batch the sums are a per-batch-entry workspace and the counts scale with the batch
    dyn = ops_body(read(emitted, "Dynamic_int8_CNN_plane_sums"))
    assert "a.out = SOFIE_I8OUT_I8_PLANE_SUMS" in dyn and "sofie_batch * 128" in dyn
    assert "sofie_hip_fill_zero(fCtx, workspace_op_" in dyn and "sofie_hip_plane_sums_to_average(" in dyn


def test_qlinear_matmul_and_conv_integer_become_one_launch_each(emitted):
    txt = read(emitted, "QLinearMatMulRelu")
    body = ops_body(txt)
    # the Relu on the int8 output rides in the GEMM's store; multipliers a_scale*b_scale[n]/y_scale are a weight
    assert body.count("sofie_hip_gemm_i8(") == 1 and "d.relu_out = 1" in body and "sofie_hip_unary_f32" not in body
    assert "tensor_P_requant_scale" in txt
    txt = read(emitted, "ConvIntegerDequantize")
    body = ops_body(txt)
    assert body.count("sofie_hip_conv_i8(") == 1 and "a.out = SOFIE_I8OUT_I32" in body and "a.relu = 1" in body
    assert "sofie_hip_dequantize_linear_i32(" in body and "sofie_hip_unary_f32" not in body


def test_qgemm_with_bias_and_relu_is_one_launch_on_an_int8_input(tmp_path):
    """The contrib operator QGemm (int8 graph input, int32 bias, per-column scales) followed by Relu: one sofie_hip_gemm_i8 with the
    bias on the accumulator and the Relu on the requantised output; the Session takes and returns int8."""
    from sofie_amd.benchsupport import models
    spec = models.int8_gemm_requant(64)
    p = str(tmp_path / "QGemmSmall.onnx")
    ow.write(p, spec["nodes"], spec["inputs"], spec["outputs"], spec["init"], name="QGemmSmall")
    em._run([em.EMIT, p, str(tmp_path)])
    txt = open(str(tmp_path / "QGemmSmall_GPU_HIP.hxx")).read()
    body = ops_body(txt)
    assert body.count("sofie_hip_gemm_i8(") == 1 and "sofie_hip_unary" not in body
    assert "d.bias = tensor_bias; d.scale = tensor_P_requant_scale;" in body
    assert "d.relu_acc = 0; d.relu_out = 1; d.out = SOFIE_I8OUT_I8; d.Y = tensor_Y;" in body
    assert re.search(r"std::vector<int8_t> infer\(int8_t const ?\* ?host_A\)", txt)
    assert "sofie_hip_transpose_i8(fCtx, packed_B, tensor_B, 64, 64, 0, 0)" in txt
    # forms the reference's parser would refuse by name are refused here too
    bad = dict(spec, nodes=[ow.node("QGemm", ["A", "sa", "zp", "B", "sb", "zp", "bias", "sy", "zp"], ["P"], alpha=0.5), spec["nodes"][1]])
    ow.write(p, bad["nodes"], bad["inputs"], bad["outputs"], bad["init"], name="QGemmSmall")
    with pytest.raises(RuntimeError, match="alpha = 1"):
        em._run([em.EMIT, p, str(tmp_path)])


def test_run_time_batch_signatures_follow_the_reference_convention(emitted):
    txt = read(emitted, "DynamicLinear")
    # the constructor takes the maximum after the weight file, infer takes the value first (core/src/RModel.cxx:1537-1547, 1375-1395)
    assert re.search(r'Session\(std::string filename = "DynamicLinear_GPU_HIP.dat", std::size_t N = 1, int device = 0\)', txt)
    assert re.search(r"std::vector<float> infer\(std::size_t N, float const ?\* ?host_X\)", txt)
    assert "void infer_nosync(std::size_t N)" in txt
    assert "sofie: dynamic input tensor shape parameter N exceeds the initialized maximum allowed shape." in txt
    assert "d.M = static_cast<std::int32_t>(sofie_batch * 1); d.N = 3; d.K = 4;" in txt
    assert "sofie_hip_upload(fCtx, tensor_X, host_X, N * 16)" in txt and "out_0(N * 3)" in txt
    assert "kArenaBytes" not in txt and "ArenaBytes(fMaxBatch)" in txt
    # shapes of the graph tensors in the reference's form: the parameter by name
    assert 'dim_X{SingleDim{"N"}, SingleDim{4}}' in txt and "inputTensorDims{makeDims(dim_X)}" in txt and "hasDynamicOutputTensors{true}" in txt
    # the int8 chain: every row count scales, the re-laid-out weights do not
    txt = read(emitted, "Dynamic_int8_MLP")
    assert txt.count("d.M = static_cast<std::int32_t>(sofie_batch * 1)") == 3
    assert "std::size_t batch_size = 1" in txt


def test_a_batch_given_at_generation_makes_a_static_session(emitted, tmp_path):
    r = subprocess.run([em.EMIT, os.path.join(emitted, "DynamicLinear.onnx"), str(tmp_path), "--batch", "4"], stdout=subprocess.PIPE,
                       stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), "DynamicLinear_GPU_HIP.hxx")).read()
    assert "sofie_batch" not in txt and "kArenaBytes" in txt and "d.M = 4; d.N = 3; d.K = 4;" in txt
    assert re.search(r"std::vector<float> infer\(float const ?\* ?host_X\)", txt)
    assert "dim_X{SingleDim{4}, SingleDim{4}}" in txt and "hasDynamicInputTensors{false}" in txt


def test_per_batch_entry_plan_scales_without_overlap(emitted, tmp_path):
    out = subprocess.run([em.EMIT, os.path.join(emitted, "Dynamic_int8_CNN.onnx"), str(tmp_path), "--plan"], check=True,
                         stdout=subprocess.PIPE, text=True).stdout.split("\n")
    head = out[1].split()
    assert head[0] == "static" and head[2] == "per_batch_entry" and head[5] == "N"
    static_bytes, entry_bytes = int(head[1]), int(head[3])
    rows = [l.split() for l in out[2:] if len(l.split()) == 7]
    per = [dict(name=f[0], offset=int(f[1]), bytes=int(f[2]), first=int(f[3]), last=int(f[4]), pooled=int(f[5])) for f in rows if f[6] == "per_batch_entry"]
    fixed = [dict(name=f[0], offset=int(f[1]), bytes=int(f[2])) for f in rows if f[6] == "static"]
    assert static_bytes % 256 == 0 and all(r["offset"] % 256 == 0 and r["offset"] + r["bytes"] <= static_bytes for r in fixed)
    names = {r["name"] for r in per}
    assert {"tensor_X", "tensor_Y", "tensor_Q", "tensor_R0", "tensor_R3"} <= names and not any(n.startswith("packed_") for n in names)
    # per-entry offsets are multiples of 16, so that capacity (a multiple of 16) times the offset is a multiple of 256
    assert all(r["offset"] % 16 == 0 and r["offset"] + r["bytes"] <= entry_bytes for r in per)
    views = [r for r in per if r["pooled"] == 2]
    assert [r["name"] for r in views] == ["tensor_F"]           # the Flatten behind the average pool: placed on its input
    for i, a in enumerate(per):
        for b in per[i + 1:]:
            if a["offset"] < b["offset"] + b["bytes"] and b["offset"] < a["offset"] + a["bytes"]:
                if 2 in (a["pooled"], b["pooled"]) and a["offset"] == b["offset"] and a["bytes"] == b["bytes"]:
                    continue    # a view and the tensor it is a view of (or another view of it)
                assert a["pooled"] and b["pooled"] and (a["last"] <= b["first"] or b["last"] <= a["first"]), (a, b)


def test_parameter_outside_the_leading_dimension_is_refused(tmp_path):
    nodes = [ow.node("Relu", ["X"], ["Y"])]
    r = _emit(tmp_path, nodes, [("X", np.float32, [4, "K"])], [("Y", np.float32, [4, "K"])], {})
    assert r.returncode != 0 and "only the leading (batch) dimension may be a parameter" in r.stdout
    # two different parameters cannot both be the batch
    nodes = [ow.node("Add", ["A", "B"], ["Y"])]
    r = _emit(tmp_path, nodes, [("A", np.float32, ["N", 4]), ("B", np.float32, ["M", 4])], [("Y", np.float32, ["N", 4])], {})
    assert r.returncode != 0 and "two shape parameters" in r.stdout
    # a transposed batched operand has no row dimension to grow
    nodes = [ow.node("Gemm", ["X", "W"], ["Y"], transA=1)]
    r = _emit(tmp_path, nodes, [("X", np.float32, ["N", 4])], [("Y", np.float32, [4, 3])], {"W": np.ones((1, 3), np.float32)})
    assert r.returncode != 0 and "run-time batch" in r.stdout


def test_view_based_infer_binds_the_callers_memory(emitted):
    txt = read(emitted, "Linear_16")
    # the operators take the graph inputs and outputs as parameters; infer_nosync binds the arena's regions,
    # the overload on views binds the caller's memory (README.md:291-297 of the reference lists the three signatures)
    assert re.search(r"void doInfer\(float const \*tensor_\w+, float \*tensor_\w+\)", txt)
    assert "void infer(std::span<ViewConstF1D const> inputs, std::span<ViewF1D> outputs)" in txt
    assert "using ViewF1D = DeviceView<float>;" in txt and "#if __cplusplus >= 202002L" in txt
    # a model whose input is not float has no such overload (the views are float views)
    assert "std::span<ViewConstF1D const>" in read(emitted, "Config5_int8_CNN_small")
    txt = read(emitted, "DynamicLinear")
    assert "void infer(std::span<ViewConstF1D const> inputs, std::span<ViewF1D> outputs, std::size_t N)" in txt


def test_one_to_one_operators_join_their_producer(emitted, tmp_path):
    body = ops_body(read(emitted, "ElementwiseChains"))
    # Gemm: LeakyRelu is its activation, Exp/Clip/Sqrt/Log ride in its store, the sixth operator is a pass of its own
    assert "d.act = SOFIE_ACT_LEAKYRELU" in body
    assert "sofie_post_ops post{4, {SOFIE_ACT_EXP, SOFIE_ACT_CLIP, SOFIE_ACT_SQRT, SOFIE_ACT_LOG}, {0.0f, 0.5f, 0.0f, 0.0f}, {0.0f, 3.0f, 0.0f, 0.0f}}; d.post = &post;" in body
    assert "sofie_hip_unary_f32(fCtx, tensor_Y, tensor_g5, 72, SOFIE_ACT_NEG" in body
    # Conv: Tanh + three links
    assert "sofie_post_ops post{3, {SOFIE_ACT_ABS, SOFIE_ACT_SOFTPLUS, SOFIE_ACT_RECIPROCAL, SOFIE_ACT_NONE}" in body
    assert "SOFIE_ACT_TANH, 0.0f, tensor_Z, &post, nullptr)" in body
    # no producer to join: chains of at most four in one pass each
    assert "sofie_post_ops ops{4, {SOFIE_ACT_SIN, SOFIE_ACT_EXP, SOFIE_ACT_ATAN, SOFIE_ACT_FLOOR}" in body
    # the chain of the reference's custom-memory model (Gemm -> Relu -> Sigmoid -> Tanh) is one launch
    body = ops_body(read(emitted, "CustomMemoryChain"))
    assert body.count("detail::Check(") == 1 and "sofie_post_ops post{2, {SOFIE_ACT_SIGMOID, SOFIE_ACT_TANH" in body
    # a graph output in the middle of a chain stops the folding there
    nodes = [ow.node("Gemm", ["X", "W"], ["G"]), ow.node("Relu", ["G"], ["R"]), ow.node("Exp", ["R"], ["Y"])]
    r = _emit(tmp_path, nodes, [("X", np.float32, [2, 3])], [("R", np.float32, [2, 4]), ("Y", np.float32, [2, 4])], {"W": np.ones((3, 4), np.float32)})
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), [f for f in os.listdir(str(tmp_path)) if f.endswith(".hxx")][0])).read()
    body = ops_body(txt)
    assert "d.act = SOFIE_ACT_RELU" in body and "d.post" not in body and "SOFIE_ACT_EXP" in body and body.count("detail::Check(") == 2


def test_equal_shaped_adds_join_the_store_of_their_producer(emitted, tmp_path):
    body = ops_body(read(emitted, "ResidualBlock"))
    # 8 operators in the graph, 3 launches: Conv(+Add+Relu), GlobalAveragePool, Gemm(+Add+Sigmoid); the Flatten is a view
    assert body.count("detail::Check(") == 3 and "sofie_hip_add_f32" not in body and "sofie_hip_unary_f32" not in body
    assert "is a view of tensor_" in body and "sofie_hip_copy(" not in body
    assert "SOFIE_ACT_RELU, 0.0f, tensor_r0, nullptr, tensor_X)" in body
    assert "d.residual = tensor_Z;" in body and "d.act = SOFIE_ACT_SIGMOID" in body
    # a broadcasting Add (bias-like operand of another shape) and an Add behind an activation stay operators of their own
    body = ops_body(read(emitted, "DynamicResidual"))
    assert body.count("sofie_hip_add_f32") == 1 and "d.residual = tensor_Z;" in body and "d.act = SOFIE_ACT_RELU" in body
    nodes = [ow.node("Gemm", ["X", "W"], ["G"]), ow.node("Relu", ["G"], ["R"]), ow.node("Add", ["R", "Z"], ["Y"])]
    r = _emit(tmp_path, nodes, [("X", np.float32, [2, 3]), ("Z", np.float32, [2, 4])], [("Y", np.float32, [2, 4])], {"W": np.ones((3, 4), np.float32)})
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), "m_GPU_HIP.hxx")).read()
    assert "d.residual" not in txt and "sofie_hip_add_f32" in txt and "d.act = SOFIE_ACT_RELU" in txt
    # the other operand must exist before the product runs: here it is computed later, so nothing is folded
    nodes = [ow.node("Gemm", ["X", "W"], ["G"]), ow.node("Tanh", ["Z"], ["T"]), ow.node("Add", ["G", "T"], ["Y"])]
    r = _emit(tmp_path, nodes, [("X", np.float32, [2, 3]), ("Z", np.float32, [2, 4])], [("Y", np.float32, [2, 4])], {"W": np.ones((3, 4), np.float32)}, name="late")
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), "late_GPU_HIP.hxx")).read()
    assert "d.residual" not in txt and "sofie_hip_add_f32" in txt


def test_corrupt_files_are_refused_with_a_message(tmp_path):
    """Damaged ONNX files end in an error message and exit status 1, never in a crash: a node without outputs, a varint that
    never ends, an initializer whose shape promises more values than the file holds, a truncated file."""
    good = ow.model([ow.node("Relu", ["X"], ["Y"])], [("X", np.float32, [1, 4])], [("Y", np.float32, [1, 4])], {"W": np.ones((2, 2), np.float32)})

    def run(data, name):
        p = os.path.join(str(tmp_path), name + ".onnx")
        open(p, "wb").write(data)
        return subprocess.run([em.EMIT, p, str(tmp_path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)

    assert run(good, "good").returncode == 0
    r = run(ow.model([ow.node("Relu", ["X"], [])], [("X", np.float32, [1, 4])], [("Y", np.float32, [1, 4])], {}), "no_output")
    assert r.returncode == 1 and "0 outputs" in r.stdout
    r = run(ow.model([ow.node("Gemm", ["X"], ["Y"])], [("X", np.float32, [1, 4])], [("Y", np.float32, [1, 4])], {}), "one_input")
    assert r.returncode == 1 and "at least 2" in r.stdout
    r = run(b"\x08" + b"\xff" * 12, "varint")
    assert r.returncode == 1 and "varint" in r.stdout
    for cut in (1, len(good) // 3, len(good) - 3):
        r = run(good[:cut], "cut%d" % cut)
        assert r.returncode in (0, 1) and (r.returncode == 0 or "error" in r.stdout)
    # the shape of the initializer claims 2^50 values
    t = ow._vi(1, 1 << 50) + ow._vi(1, 2) + ow._vi(2, 1) + ow._ld(8, b"W") + ow._ld(9, np.ones(4, np.float32).tobytes())
    g = ow._ld(1, ow.node("Relu", ["X"], ["Y"])) + ow._ld(2, b"g") + ow._ld(5, t) + ow._ld(11, ow.value_info("X", 1, [1, 4])) + ow._ld(12, ow.value_info("Y", 1, [1, 4]))
    r = run(ow._vi(1, 8) + ow._ld(7, g), "huge")
    assert r.returncode == 1 and ("2^40" in r.stdout or "values" in r.stdout)


def test_packed_fields_wire_types_and_float_lists(tmp_path):
    """The packed-integer decoder holds varints to 10 bytes like the plain one; a string field written as a varint is a malformed
    file, not a null string; `floats` attributes (packed or one fixed32 each) are read, so a Constant given as value_floats becomes
    an initializer."""
    def run(data, name):
        p = os.path.join(str(tmp_path), name + ".onnx")
        open(p, "wb").write(data)
        return subprocess.run([em.EMIT, p, str(tmp_path), "--name", name], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)

    def graph(node_bytes, extra=b""):
        g = ow._ld(1, node_bytes) + ow._ld(2, b"g") + extra + ow._ld(11, ow.value_info("X", 1, [1, 4])) + ow._ld(12, ow.value_info("Y", 1, [1, 4]))
        return ow._vi(1, 8) + ow._ld(8, ow._ld(2, ow._vi(2, 17))) + ow._ld(7, g)

    # an `ints` attribute whose packed payload is one varint of 12 continuation bytes
    bad_ints = ow._ld(1, b"axes") + ow._ld(8, b"\xff" * 12 + b"\x01") + ow._vi(20, 7)
    n = ow._ld(1, b"X") + ow._ld(2, b"Y") + ow._ld(4, b"Relu") + ow._ld(5, bad_ints)
    r = run(graph(n), "overlong")
    assert r.returncode == 1 and "varint longer than 10 bytes" in r.stdout
    # the operator type (field 4, a string) written as a varint
    n = ow._ld(1, b"X") + ow._ld(2, b"Y") + ow._vi(4, 7)
    r = run(graph(n), "mistyped")
    assert r.returncode == 1 and "length-delimited" in r.stdout
    # Constant(value_floats) -> Add: the constant is an initializer of the generated Session, packed and unpacked encodings alike
    import struct
    vals = [0.5, -1.25, 3.0, 8.0]
    for name, payload in (("packed", ow._ld(7, struct.pack("<4f", *vals))), ("unpacked", b"".join(ow._key(7, 5) + struct.pack("<f", v) for v in vals))):
        const = ow._ld(2, b"C") + ow._ld(4, b"Constant") + ow._ld(5, ow._ld(1, b"value_floats") + payload + ow._vi(20, 6))
        add = ow.node("Add", ["X", "C"], ["Y"])
        g = ow._ld(1, const) + ow._ld(1, add) + ow._ld(2, b"g") + ow._ld(11, ow.value_info("X", 1, [1, 4])) + ow._ld(12, ow.value_info("Y", 1, [1, 4]))
        r = run(ow._vi(1, 8) + ow._ld(8, ow._ld(2, ow._vi(2, 17))) + ow._ld(7, g), "floats_" + name)
        assert r.returncode == 0, r.stdout
        dat = open(os.path.join(str(tmp_path), "floats_%s_GPU_HIP.dat" % name)).read().split()
        assert dat[0] == "tensor_C" and dat[1] == "4" and [float(v) for v in dat[2:6]] == vals


def test_parse_time_rewrites_of_the_reference(emitted, tmp_path):
    txt = read(emitted, "ParseRewrites")
    body = ops_body(txt)
    # 11 nodes, 4 launches: Cast aliased, both Transposes absorbed as transA / transB, MatMul + Add -> Gemm with bias,
    # the Gemm of weights folded (with its Relu) into a constant, Conv + Add(1-D initializer) -> Conv with bias
    assert body.count("detail::Check(") == 4
    assert "d.transA = 0; d.transB = 1;" in body and "d.A = tensor_X; d.B = tensor_W2; d.C = tensor_b1; d.bias_mode = SOFIE_BIAS_ROW;" in body
    assert "d.transA = 1; d.transB = 0;" in body and "d.A = tensor_A2;" in body
    assert "computed when the code was generated" in body and "tensor_Kr" in txt and "static const float host[12]" in txt
    assert "tensor_I, tensor_Wc, tensor_cb, SOFIE_ACT_NONE" in body
    assert "Transpose" not in body and "Cast" not in body
    assert "-> K2: a product of weights" in body and "-> Ks: constants only" in body and "d.residual" not in body
    # a Cast that changes the type is not rewritten away: it is refused by name
    r = _emit(tmp_path, [ow.node("Cast", ["X"], ["Y"], to=7)], [("X", np.float32, [1, 4])], [("Y", np.int64, [1, 4])], {})
    assert r.returncode != 0 and "Cast" in r.stdout
    # a Transpose that is also a graph output stays an operator of its own (a gather kernel), and the MatMul reads its result
    r = _emit(tmp_path, [ow.node("Transpose", ["X"], ["T"]), ow.node("MatMul", ["T", "W"], ["Y"])], [("X", np.float32, [3, 2])],
              [("T", np.float32, [2, 3]), ("Y", np.float32, [2, 4])], {"W": np.ones((3, 4), np.float32)}, name="kept")
    kept = open(os.path.join(str(tmp_path), "kept_GPU_HIP.hxx")).read()
    assert r.returncode == 0 and "sofie_hip_transpose_f32(" in kept and "d.A = tensor_T;" in kept and "d.transA = 0;" in kept


def test_asymmetric_zero_point_is_refused(tmp_path):
    init = {"W": np.ones((4, 3, 1, 1), dtype=np.int8), "s": np.array(0.5, dtype=np.float32), "z": np.zeros((), dtype=np.int8),
            "z1": np.array(3, dtype=np.int8), "sx": np.array(0.1, dtype=np.float32)}
    nodes = [ow.node("QuantizeLinear", ["X", "sx", "z"], ["Q"]),
             ow.node("QLinearConv", ["Q", "s", "z1", "W", "s", "z", "s", "z"], ["Y"], kernel_shape=[1, 1], pads=[0, 0, 0, 0])]
    r = _emit(tmp_path, nodes, [("X", np.float32, [1, 3, 4, 4])], [("Y", np.int8, [1, 4, 4, 4])], init)
    assert r.returncode != 0 and "zero point" in r.stdout


def test_custom_memory_header_allocates_nothing(emitted):
    # the counterpart of the reference's GeneratedCodeHasNoAlpakaDeviceAllocation (tests/alpaka/TestAlpakaCustomMemory.cxx:103-111)
    for model in ("CustomMemoryChain", "CustomMemoryStreamChain"):
        txt = read(emitted, model)
        assert "sofie_hip_arena_create" not in txt and "sofie_hip_arena_adopt(fCtx, fBlock, kArenaBytes)" in txt
        assert "struct MemoryProvider" in txt and "Session(MemoryProvider provider, std::string filename" in txt
    assert "void *stream = nullptr" in read(emitted, "CustomMemoryStreamChain")


# ---- safetensors weights (the reference's Options::kSafetensorsWeightFile; its tests: tests/cpu/TestSafetensorsWeights.cxx) ----

def _run_session(emitted, model, weights_path):
    lib = ctypes.CDLL(os.path.join(emitted, "lib%s.so" % model))
    err = ctypes.create_string_buffer(1024)
    x = np.ones(1600, dtype=np.float32)
    y = np.zeros(160, dtype=np.float32)
    inp = (ctypes.c_void_p * 1)(x.ctypes.data)
    rc = lib.run_model(str(weights_path).encode(), inp, y.ctypes.data_as(ctypes.c_void_p), ctypes.c_ulong(160), err, 1024)
    return rc, err.value.decode(), y


def test_safetensors_file_is_read_by_the_safetensors_library(emitted):
    from safetensors.numpy import load_file
    from tests import onnx_lite
    got = load_file(os.path.join(emitted, "Linear_16_st_GPU_HIP.safetensors"))
    g = onnx_lite.load(os.path.join(em.GOLDEN, "models", "Linear_16.onnx"))
    assert len(got) == len(g["initializers"])
    for k, v in g["initializers"].items():
        key = "tensor_" + re.sub(r"[^A-Za-z0-9_]", "_", k)
        assert got[key].dtype == np.float32 and got[key].shape == np.asarray(v).shape
        assert np.array_equal(got[key].view(np.uint32), np.asarray(v, dtype=np.float32).view(np.uint32)), k


def test_safetensors_payload_is_validated_before_any_device_work(emitted, tmp_path):
    """Every inconsistency of the payload is reported by name, and a payload that passes goes on to the device
    (which this machine may not have: then the error is the runtime's, not the reader's)."""
    import torch
    from safetensors.numpy import load_file, save_file
    good = load_file(os.path.join(emitted, "Linear_16_st_GPU_HIP.safetensors"))

    def attempt(tensors, **kw):
        path = tmp_path / "w.safetensors"
        save_file(tensors, str(path), **kw)
        return _run_session(emitted, "Linear_16_st", path)

    rc, msg, _ = _run_session(emitted, "Linear_16_st", tmp_path / "missing.safetensors")
    assert rc == 1 and "failed to open file" in msg
    missing = dict(good)
    del missing["tensor_18_bias"]
    rc, msg, _ = attempt(missing)
    assert rc == 1 and "tensor_18_bias is missing" in msg
    wrong_type = dict(good)
    wrong_type["tensor_0_bias"] = good["tensor_0_bias"].astype(np.float64)
    rc, msg, _ = attempt(wrong_type)
    assert rc == 1 and "tensor_0_bias has dtype F64" in msg
    wrong_size = dict(good)
    wrong_size["tensor_0_weight"] = good["tensor_0_weight"][:-1]
    rc, msg, _ = attempt(wrong_size)
    assert rc == 1 and "tensor_0_weight has" in msg and "elements" in msg
    raw = open(os.path.join(emitted, "Linear_16_st_GPU_HIP.safetensors"), "rb").read()
    for name, blob, text in (("short", raw[:5], "shorter than"), ("cut", raw[:8] + raw[8:40], "exceeds the payload"),
                             ("payload", raw[:-100], "data offsets"), ("json", raw[:8] + b"[" + raw[9:], "malformed header")):
        p = tmp_path / (name + ".safetensors")
        p.write_bytes(blob)
        rc, msg, _ = _run_session(emitted, "Linear_16_st", p)
        assert rc == 1 and text in msg, (name, msg)
    # a file written by the safetensors library itself (other key order, spaces, a __metadata__ entry) passes the reader
    rc, msg, _ = attempt(dict(reversed(list(good.items()))), metadata={"producer": "test"})
    if not torch.cuda.is_available():
        assert rc == 1 and "SOFIE HIP runtime error in Session" in msg


def test_pool_attributes_resolve_to_the_reference_shapes(emitted, tmp_path):
    """Output extents of the reference's shape inference (ROperator_Pool.hxx:107-171) as they appear in the emitted call."""
    def emit_pool(op, shape, name, **attrs):
        r = _emit(tmp_path, [ow.node(op, ["X"], ["Y"], **attrs)], [("X", np.float32, shape)], [("Y", np.float32, shape)], {}, name=name)
        return r, (open(os.path.join(str(tmp_path), name + "_GPU_HIP.hxx")).read() if r.returncode == 0 else "")
    # the reference's own test shapes: 6 -> 2 (MaxPool1d_CeilMode_Overhang), 5x5 -> 3x3 (MaxPool2d_CeilMode), 4x4 -> 3x5 (AsymPad)
    r, txt = emit_pool("MaxPool", [1, 1, 6], "overhang", kernel_shape=[2], strides=[3], ceil_mode=1)
    assert r.returncode == 0 and "d.H = 1; d.W = 6; d.OH = 1; d.OW = 2;" in txt and "SOFIE_POOL_MAX" in txt
    r, txt = emit_pool("MaxPool", [1, 1, 5, 5], "ceil2d", kernel_shape=[2, 2], strides=[2, 2], ceil_mode=1)
    assert r.returncode == 0 and "d.OH = 3; d.OW = 3;" in txt
    r, txt = emit_pool("MaxPool", [1, 1, 4, 4], "asym", kernel_shape=[2, 2], pads=[0, 1, 0, 1], strides=[1, 1])
    assert r.returncode == 0 and "d.OH = 3; d.OW = 5;" in txt and "d.pad_h0 = 0; d.pad_w0 = 1; d.pad_h1 = 0; d.pad_w1 = 1;" in txt
    # SAME_UPPER puts the odd sample at the end; without padding and ceil_mode the divisor is the constant kh*kw
    r, txt = emit_pool("AveragePool", [2, 3, 7, 7], "same", kernel_shape=[2, 2], strides=[2, 2], auto_pad="SAME_UPPER", count_include_pad=1)
    assert r.returncode == 0 and "d.OH = 4; d.OW = 4;" in txt and "d.pad_h0 = 0; d.pad_w0 = 0; d.pad_h1 = 1; d.pad_w1 = 1;" in txt
    assert "d.count_include_pad = 1; d.dynamic_divisor = 1;" in txt and "d.planes = 6;" in txt
    r, txt = emit_pool("AveragePool", [2, 3, 8, 8], "plain", kernel_shape=[2, 2], strides=[2, 2])
    assert r.returncode == 0 and "d.dynamic_divisor = 0;" in txt
    # three spatial axes are one call with the axes slowest first: {in}, {out}, {window}, {pad begin}, {pad end}, {stride}
    r, txt = emit_pool("MaxPool", [1, 2, 4, 5, 6], "three_d", kernel_shape=[2, 2, 3], strides=[2, 1, 3], pads=[0, 1, 0, 0, 0, 0])
    assert r.returncode == 0 and "sofie_pool3d_desc d{2, {4, 5, 6}, {2, 5, 2}, {2, 2, 3}, {0, 1, 0}, {0, 0, 0}, {2, 1, 3}, SOFIE_POOL_MAX, 0, 1};" in txt
    # refusals name the operator
    r, _ = emit_pool("MaxPool", [1, 1, 4, 4, 4, 4], "four_d", kernel_shape=[2, 2, 2, 2])
    assert r.returncode != 0 and "MaxPool" in r.stdout and "spatial" in r.stdout
    r, _ = emit_pool("MaxPool", [1, 1, 4, 4], "column_major", kernel_shape=[2, 2], storage_order=1)
    assert r.returncode != 0 and "storage_order" in r.stdout
    r, _ = emit_pool("AveragePool", [1, 1, 4, 4], "too_big", kernel_shape=[6, 6])
    assert r.returncode != 0 and "larger than the padded input" in r.stdout
    r = _emit(tmp_path, [ow.node("MaxPool", ["X"], ["Y", "I"], kernel_shape=[2, 2])], [("X", np.float32, [1, 1, 4, 4])],
              [("Y", np.float32, [1, 1, 3, 3])], {}, name="indices")
    assert r.returncode != 0 and "Indices" in r.stdout


def test_reduce_shapes_axes_and_refusals(tmp_path):
    f = np.float32
    # keepdims = 0 over the two middle axes, the axes as an input; negative axes; everything reduced when no axes are given
    r = _emit(tmp_path, [ow.node("ReduceSum", ["X", "ax"], ["Y"], keepdims=0), ow.node("ReduceMean", ["X"], ["Z"], axes=[-1]), ow.node("ReduceProd", ["X"], ["P"], keepdims=0)],
              [("X", f, [2, 3, 4, 5])], [("Y", f, [2, 5]), ("Z", f, [2, 3, 4, 1]), ("P", f, [])], {"ax": np.array([1, 2], np.int64)}, name="red")
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), "red_GPU_HIP.hxx")).read()
    assert "tensor_X, 2, 12, 5, SOFIE_REDUCE_SUM)" in txt and "tensor_X, 24, 5, 1, SOFIE_REDUCE_MEAN)" in txt and "tensor_X, 1, 120, 1, SOFIE_REDUCE_PROD)" in txt
    # axes that are not adjacent, an axis out of range, axes computed at run time
    r = _emit(tmp_path, [ow.node("ReduceMax", ["X"], ["Y"], axes=[0, 2])], [("X", f, [2, 3, 4])], [("Y", f, [1, 3, 1])], {}, name="gap")
    assert r.returncode != 0 and "ReduceMax" in r.stdout and "not adjacent" in r.stdout
    r = _emit(tmp_path, [ow.node("ReduceMin", ["X"], ["Y"], axes=[3])], [("X", f, [2, 3, 4])], [("Y", f, [2, 3, 4])], {}, name="range")
    assert r.returncode != 0 and "invalid axes values 3" in r.stdout
    r = _emit(tmp_path, [ow.node("ReduceL2", ["X", "A"], ["Y"])], [("X", f, [2, 3]), ("A", np.int64, [1])], [("Y", f, [2, 1])], {}, name="runtime_axes")
    assert r.returncode != 0 and "int64 initializer" in r.stdout


def test_indexing_operators_shapes_and_refusals(tmp_path):
    f, i64 = np.float32, lambda *v: np.array(v, np.int64)
    # Slice before opset 10 (attributes), ends beyond the axis clamp; Split in unequal parts; Gather with a scalar index drops the axis
    r = _emit(tmp_path, [ow.node("Slice", ["X"], ["S"], starts=[1], ends=[1000], axes=[1]), ow.node("Split", ["X", "parts"], ["A", "B"], axis=0),
                         ow.node("Gather", ["X", "i"], ["G"], axis=1)],
              [("X", f, [4, 5])], [("S", f, [4, 4]), ("A", f, [1, 5]), ("B", f, [3, 5]), ("G", f, [4])], {"parts": i64(1, 3), "i": np.array(3, np.int64)}, name="idx")
    assert r.returncode == 0, r.stdout
    txt = open(os.path.join(str(tmp_path), "idx_GPU_HIP.hxx")).read()
    assert "shape[6] = {4, 4, 1, 1, 1, 1}" in txt and "strides, 1, 20)" in txt and "strides, 5, 20)" in txt and "+ 12, 20, 4, 4)" in txt
    for nodes, init, words in [
            ([ow.node("Slice", ["X", "s", "e"], ["Y"])], {"s": i64(2), "e": i64(2)}, "empty"),
            ([ow.node("Slice", ["X", "s", "e", "a", "t"], ["Y"])], {"s": i64(0), "e": i64(2), "a": i64(0), "t": i64(0)}, "step 0"),
            ([ow.node("Split", ["X", "p"], ["Y", "Z"])], {"p": i64(1, 2)}, "Sum of split sizes"),
            ([ow.node("Expand", ["X", "p"], ["Y"])], {"p": i64(3, 5)}, "cannot be broadcast"),
            ([ow.node("Tile", ["X", "p"], ["Y"])], {"p": i64(2)}, "one repeat per axis"),
            ([ow.node("Gather", ["X", "p"], ["Y"])], {"p": i64(4)}, "index 4 is out of range"),
            ([ow.node("Gather", ["X", "X2"], ["Y"])], {}, "int64 initializer")]:
        r = _emit(tmp_path, nodes, [("X", f, [4, 5]), ("X2", f, [4, 5])], [("Y", f, [4, 5])], init, name="bad")
        assert r.returncode != 0 and words in r.stdout, (words, r.stdout)


def test_constant_nodes_become_initializers(tmp_path):
    """Exporters hand Reshape its shape, Slice its bounds and a Gemm its weights through Constant nodes: the parser registers each as an initializer
    under the node's output name (parsers/src/ParseConstant.cxx), so the emitted code equals that of the same graph with initializers."""
    f = np.float32
    W = np.arange(12, dtype=f).reshape(4, 3)
    nodes = [ow.node("Constant", [], ["W"], value=W), ow.node("Constant", [], ["shape"], value=np.array([2, 6], np.int64)),
             ow.node("Constant", [], ["st"], value_ints=[1]), ow.node("Constant", [], ["en"], value_ints=[3]),
             ow.node("MatMul", ["X", "W"], ["Y"]), ow.node("Reshape", ["Y", "shape"], ["R"]), ow.node("Slice", ["R", "st", "en"], ["S"])]
    r = _emit(tmp_path, nodes, [("X", f, [4, 4])], [("S", f, [1, 6])], {}, name="viaconst")
    assert r.returncode == 0, r.stdout
    a = open(os.path.join(str(tmp_path), "viaconst_GPU_HIP.hxx")).read()
    same = [n for n in nodes if n not in nodes[:4]]
    r = _emit(tmp_path, same, [("X", f, [4, 4])], [("S", f, [1, 6])], {"W": W, "shape": np.array([2, 6], np.int64), "st": np.array([1], np.int64), "en": np.array([3], np.int64)},
              name="viainit")
    assert r.returncode == 0, r.stdout
    b = open(os.path.join(str(tmp_path), "viainit_GPU_HIP.hxx")).read()
    assert ops_body(a) == ops_body(b) and "sofie_hip_strided_gather_f32" in a and "strides, 6, 12)" in a
    assert open(os.path.join(str(tmp_path), "viaconst_GPU_HIP.dat")).read().split()[-12:] == open(os.path.join(str(tmp_path), "viainit_GPU_HIP.dat")).read().split()[-12:]
    r = _emit(tmp_path, [ow.node("Constant", [], ["W"]), ow.node("Relu", ["X"], ["Y"])], [("X", f, [4])], [("Y", f, [4])], {}, name="novalue")
    assert r.returncode != 0 and "has no value" in r.stdout

"""Sessions whose batch is a run-time parameter: the constructor takes the maximum, every infer call the batch
(the reference's convention, core/src/RModel.cxx:1375-1395, 1537-1547; its tests: tests/alpaka/TestAlpakaLinear.cxx:121-210).
One Session serves several batch sizes; each result is compared with the CPU oracle on the same rows."""
import ctypes
import os

import numpy as np
import pytest

from sofie_amd import runtime as R
from tests import emitted_models as em
from tests import graph_runner as gr
from tests import onnx_lite
from tests import util

pytestmark = pytest.mark.gpu


class DynamicSession:
    def __init__(self, model, max_batch):
        path = os.path.join(em.OUT, "lib%s.so" % model)
        assert os.path.exists(path), "emitted models are built by __graft_entry__.build()"
        self.lib = ctypes.CDLL(path)
        self.lib.dyn_open.restype = ctypes.c_void_p
        self.lib.dyn_open.argtypes = [ctypes.c_char_p, ctypes.c_ulong, ctypes.c_char_p, ctypes.c_int]
        self.lib.dyn_close.argtypes = [ctypes.c_void_p]
        self.lib.dyn_infer.restype = ctypes.c_long
        self.lib.dyn_infer.argtypes = [ctypes.c_void_p, ctypes.c_ulong, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_ulong, ctypes.c_char_p, ctypes.c_int]
        self.lib.arena_bytes.restype = ctypes.c_ulong
        self.lib.arena_bytes.argtypes = [ctypes.c_ulong]
        self.lib.pool_bytes.restype = ctypes.c_ulong
        self.lib.pool_bytes.argtypes = [ctypes.c_void_p]
        self.err = ctypes.create_string_buffer(1024)
        print("dynamic session", model, "max batch", max_batch, flush=True)
        self.h = self.lib.dyn_open(os.path.join(em.OUT, model + "_GPU_HIP.dat").encode(), max_batch, self.err, 1024)
        assert self.h, self.err.value.decode()

    def infer(self, batch, inputs, capacity):
        arrs = [np.ascontiguousarray(a, dtype=np.float32) for a in inputs]
        ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
        y = np.zeros(capacity, dtype=np.float32)
        n = self.lib.dyn_infer(self.h, batch, ptrs, y.ctypes.data_as(ctypes.c_void_p), capacity, self.err, 1024)
        if n < 0:
            raise RuntimeError(self.err.value.decode())
        return y[:n]

    def close(self):
        if self.h:
            self.lib.dyn_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()


def test_dynamic_linear_as_the_reference_tests_it(rt):
    c = em.dynamic_linear()["consts"]
    for n in (1, 8):
        x = ((np.arange(n * 4) % 7).astype(np.float32) - 3.0).reshape(n, 4)
        want = np.maximum(x.astype(np.float64) @ c["W"].astype(np.float64) + c["B"], 0)
        with DynamicSession("DynamicLinear", n) as s:
            got = s.infer(n, [x], n * 3)
        assert got.size == n * 3 and np.abs(got.reshape(n, 3) - want).max() <= 1e-5


def test_dynamic_matmul_with_both_operands_batched(rt):
    M, K, Nc = 4, 8, 6
    for n in (1, 5):
        a = (((np.arange(n * M * K) % 11).astype(np.float32) - 5.0) * np.float32(0.3)).reshape(n, M, K)
        b = (((np.arange(n * K * Nc) % 7).astype(np.float32) - 3.0) * np.float32(0.5)).reshape(n, K, Nc)
        want = np.matmul(a.astype(np.float64), b.astype(np.float64))
        with DynamicSession("DynamicMatMulBatched", n) as s:
            got = s.infer(n, [a, b], n * M * Nc)
        assert np.abs(got.reshape(n, M, Nc) - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_one_session_serves_several_batches_and_refuses_more_than_its_maximum(rt):
    c = em.dynamic_linear()["consts"]
    x = util.normal(8101, 8 * 4).reshape(8, 4)
    want = np.maximum(x @ c["W"] + c["B"], 0).astype(np.float32)
    with DynamicSession("DynamicLinear", 8) as s:
        first = s.infer(8, [x], 24).copy()
        assert np.abs(first.reshape(8, 3) - want).max() <= 1e-5
        small = s.infer(3, [x[:3]], 24)
        assert small.size == 9 and np.array_equal(small, first[:9])
        assert s.infer(0, [x], 24).size == 0
        again = s.infer(8, [x], 24)
        assert np.array_equal(again, first)
        with pytest.raises(RuntimeError, match="dynamic input tensor shape parameter N exceeds the initialized maximum allowed shape"):
            s.infer(9, [np.zeros((9, 4), np.float32)], 27)
        # the arena grows in steps of 16 batch entries and linearly beyond
        a = [s.lib.arena_bytes(n) for n in (1, 16, 17, 32, 48)]
        assert a[0] == a[1] < a[2] == a[3] < a[4] and a[4] - a[3] == a[3] - a[1]


def test_dynamic_int8_mlp_is_bit_exact_for_every_batch(rt):
    from oracle import binding as ob
    spec = em.int8_mlp([64, 128, 96, 32], 48)
    c, x = spec["consts"], spec["feeds"][0]
    with DynamicSession("Dynamic_int8_MLP", 48) as s:
        for n in (48, 1, 17, 48):
            h = x[:n]
            for l, w in enumerate(c["weights"]):
                q = ob.quantize_linear(h, c["in_scales"][l])
                acc = np.maximum(ob.matmul_integer(q, w, M=n, N=w.shape[1], K=w.shape[0], omp=True), 0)
                h = ob.dequantize_linear(acc, np.float32(c["in_scales"][l] * c["w_scales"][l]))
            print("Dynamic_int8_MLP batch", n, flush=True)
            got = s.infer(n, [x[:n]], 48 * 32)
            assert got.size == h.size and np.array_equal(got.view(np.uint32), h.ravel().view(np.uint32))
            assert np.abs(h).max() > 0


def test_dynamic_int8_cnn_matches_cpu_chain_for_every_batch(rt):
    from tests.refmodels import int8_cnn_oracle
    spec = em.int8_cnn(2, 12)
    x = np.concatenate([spec["feeds"][0], util.normal(8201, 3 * 3 * 12 * 12).reshape(3, 3, 12, 12)])
    with DynamicSession("Dynamic_int8_CNN", 5) as s:
        assert s.lib.pool_bytes(s.h) > 0
        for n in (5, 2, 1, 5):
            want = int8_cnn_oracle(spec["consts"], x[:n]).ravel()
            print("Dynamic_int8_CNN batch", n, flush=True)
            got = s.infer(n, [x[:n]], 50)
            assert got.size == want.size == n * 10
            assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
            assert np.abs(want).max() > 1e-3


def test_dynamic_int8_cnn_with_plane_sums_for_every_batch(rt):
    from tests.refmodels import int8_cnn_oracle
    spec = em.int8_cnn(2, 16, (3, 64, 128))
    x = np.concatenate([spec["feeds"][0], util.uniform01(8202, 3 * 3 * 16 * 16).reshape(3, 3, 16, 16)])
    with DynamicSession("Dynamic_int8_CNN_plane_sums", 5) as s:
        for n in (5, 2, 1, 5):
            want = int8_cnn_oracle(spec["consts"], x[:n]).ravel()
            print("Dynamic_int8_CNN_plane_sums batch", n, flush=True)
            got = s.infer(n, [x[:n]], 50)
            assert got.size == want.size == n * 10
            assert np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))
            assert np.abs(want).max() > 1e-3


def test_dynamic_shape_plumbing(rt):
    spec = em.shape_plumbing(3)
    x = np.concatenate([spec["feeds"][0], util.normal(8304, 2 * 24).reshape(2, 2, 3, 4)])
    z = np.concatenate([spec["feeds"][1], util.normal(8305, 2 * 6).reshape(2, 3, 2)])
    with DynamicSession("Dynamic_ShapePlumbing", 5) as s:
        for n in (5, 3, 1):
            # the static model's Reshape keeps the batch through its leading 0, so the same graph evaluates any batch on the CPU
            g = onnx_lite.load(os.path.join(em.OUT, "ShapePlumbing.onnx"))
            want = gr.run(g, [x[:n], z[:n]], gr.OracleBackend()).ravel()
            print("Dynamic_ShapePlumbing batch", n, flush=True)
            got = s.infer(n, [x[:n], z[:n]], want.size)
            assert got.size == want.size == n * 6 and np.abs(got - want).max() <= 1e-5 * max(1.0, float(np.abs(want).max()))


def test_dynamic_reduce_block_keeps_or_consumes_the_batch(rt):
    from oracle import binding as ob
    x = np.concatenate([em.reduce_block(3)["feeds"][0], util.normal(8306, 4 * 24).reshape(4, 4, 6)])
    with DynamicSession("Dynamic_ReduceBlock", 7) as s:
        for n in (7, 3, 1):
            X = x[:n]
            C = ob.binary_broadcast(X, ob.reduce(X, R.REDUCE_MEAN, [2], 1), 1)
            # Y1 and Y2 keep the batch; Y3 sums over it (the reference's DynamicReduceMaxFirst reduces over the run-time dimension in the same way)
            want = np.concatenate([ob.reduce(C, R.REDUCE_L2, [-1], 0).ravel(), ob.reduce(X, R.REDUCE_MAX, [1], 0).ravel(), ob.reduce(X, R.REDUCE_SUM, [0], 1).ravel()])
            print("Dynamic_ReduceBlock batch", n, flush=True)
            got = s.infer(n, [X], want.size)
            assert got.size == want.size == n * 10 + 24 and np.array_equal(got, want)


def test_dynamic_indexing_block(rt):
    from tests.test_gpu_emitted import indexing_block_expected
    x = np.concatenate([em.indexing_block(3)["feeds"][0], util.normal(8307, 2 * 48).reshape(2, 6, 8)])
    with DynamicSession("Dynamic_IndexingBlock", 5) as s:
        for n in (5, 2, 1):
            want = indexing_block_expected(x[:n])
            print("Dynamic_IndexingBlock batch", n, flush=True)
            got = s.infer(n, [x[:n]], want.size)
            assert got.size == want.size and np.array_equal(got, want)


def test_dynamic_softmax_head(rt):
    spec = em.softmax_head(4)
    g = onnx_lite.load(os.path.join(em.OUT, "ClassifierHead.onnx"))     # the same weights with a fixed batch
    x = np.concatenate([spec["feeds"][0], util.normal(8303, 5 * 20).reshape(5, 20)])
    want = gr.run(g, [x], gr.OracleBackend(), all_outputs=True)[0]
    with DynamicSession("Dynamic_SoftmaxHead", 9) as s:
        for n in (9, 4, 1):
            print("Dynamic_SoftmaxHead batch", n, flush=True)
            got = s.infer(n, [x[:n]], want.size)
            w = want[:n].ravel()
            assert got.size == w.size and np.all(np.abs(got - w) <= 1e-5 * w + 1e-7)


def test_dynamic_conv_batchnorm_relu(rt):
    spec = em.conv_batchnorm_relu(2)
    g = onnx_lite.load(os.path.join(em.OUT, "ConvBatchNormRelu.onnx"))     # the same weights with a fixed batch of 2
    x2 = spec["feeds"][0]
    x = np.concatenate([x2, util.normal(8301, x2[:1].size).reshape(x2[:1].shape)])
    want = gr.run(g, [x], gr.OracleBackend())
    with DynamicSession("Dynamic_ConvBatchNormRelu", 3) as s:
        for n in (3, 1):
            print("Dynamic_ConvBatchNormRelu batch", n, flush=True)
            got = s.infer(n, [x[:n]], want.size)
            w = want[:n].ravel()
            assert got.size == w.size and np.abs(got - w).max() <= 1e-5 * max(1.0, float(np.abs(w).max()))


def test_dynamic_conv_pool_stack(rt):
    spec = em.conv_pool_stack(2)
    g = onnx_lite.load(os.path.join(em.OUT, "ConvPoolStack.onnx"))     # the same weights with a fixed batch of 2
    x2 = spec["feeds"][0]
    x = np.concatenate([x2, util.normal(8302, 3 * x2[:1].size).reshape((3,) + x2.shape[1:])])
    want = gr.run(g, [x], gr.OracleBackend())
    with DynamicSession("Dynamic_ConvPoolStack", 5) as s:
        for n in (5, 2, 1):
            print("Dynamic_ConvPoolStack batch", n, flush=True)
            got = s.infer(n, [x[:n]], want.size)
            w = want[:n].ravel()
            assert got.size == w.size and np.abs(got - w).max() <= 1e-5 * max(1.0, float(np.abs(w).max()))


def test_dynamic_batch_through_broadcasting_adds(rt):
    c = em.dynamic_residual()["consts"]
    x, z = util.normal(8401, 9 * 6).reshape(9, 6), util.normal(8402, 9 * 5).reshape(9, 5)
    with DynamicSession("DynamicResidual", 9) as s:
        for n in (9, 4, 1):
            want = np.maximum(x[:n].astype(np.float64) @ c["W"].astype(np.float64) + z[:n], 0) + c["b"]
            got = s.infer(n, [x[:n], z[:n]], 45)
            assert got.size == n * 5 and np.abs(got.reshape(n, 5) - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_dynamic_fp8_gemm_within_the_stated_bound(rt):
    from oracle import binding as ob
    K, N = 256, 96
    s, w8 = 2024, np.empty(N * K, dtype=np.uint8)
    for i in range(N * K):                      # the code sequence of sofie_amd/emit/tools/emit_example_api.cxx
        s = (s * 1664525 + 1013904223) & 0xFFFFFFFF
        w8[i] = (s >> 24) & 0xBE
    w8 = w8.reshape(N, K)
    bias = (0.25 * ((np.arange(N) % 7) - 3)).astype(np.float32)
    x = util.normal(8501, 40 * K).reshape(40, K)
    xs, wsc = np.float32(0.03125), np.float32(0.0078125)
    with DynamicSession("ApiDynamicFp8Gemm", 40) as sess:
        for n in (40, 7):
            a8 = ob.quantize_fp8(x[:n], xs)
            want, abs_sum = ob.gemm_fp8(a8, w8, M=n, N=N, K=K, transB=1, bias=bias, scale=np.float32(xs * wsc), act=4, out=1, want_abs_sum=True)
            got = sess.infer(n, [x[:n]], 40 * N).reshape(n, N)
            bound = 1.2 * 2.0 ** -14 * abs_sum.astype(np.float64) * float(xs * wsc) + 1e-6     # the bound of the static FP8 test
            assert np.all(np.abs(got.astype(np.float64) - want) <= bound) and np.abs(want).max() > 0.5


def test_dynamic_residual_block(rt):
    spec = em.residual_block(2)
    g = onnx_lite.load(os.path.join(em.OUT, "ResidualBlock.onnx"))
    x = np.concatenate([spec["feeds"][0], util.normal(8601, 3 * 8 * 6 * 6).reshape(3, 8, 6, 6)])
    z = np.concatenate([spec["feeds"][1], util.normal(8602, 3 * 4).reshape(3, 4)])
    with DynamicSession("Dynamic_ResidualBlock", 5) as s:
        for n in (5, 2):
            want = gr.run(g, [x[:n], z[:n]], gr.OracleBackend()).ravel()
            got = s.infer(n, [x[:n], z[:n]], 20)
            assert got.size == want.size == n * 4 and np.abs(got - want).max() <= 1e-5


def test_reset_state_and_weights_to_zero(rt):
    """resetState zeroes the pool of intermediates (the next inference is unaffected), SetWeightsToZero the float weights
    (core/src/RModel_ALPAKA.cxx:1543-1568, core/src/RModel.cxx:1632-1643)."""
    spec = em.int8_cnn(2, 12)
    x = spec["feeds"][0]
    with DynamicSession("Dynamic_int8_CNN", 2) as s:
        s.lib.dyn_maintenance.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p, ctypes.c_int]
        s.lib.pool_statistics.restype = ctypes.c_double
        s.lib.pool_statistics.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_ulong), ctypes.POINTER(ctypes.c_ulong)]
        first = s.infer(2, [x], 20).copy()
        assert s.lib.dyn_maintenance(s.h, 0, s.err, 1024) == 0, s.err.value.decode()
        assert np.array_equal(s.infer(2, [x], 20), first)
        free, largest = ctypes.c_ulong(), ctypes.c_ulong()
        frag = s.lib.pool_statistics(s.h, ctypes.byref(free), ctypes.byref(largest))
        assert 0.0 <= frag < 1.0 and largest.value <= free.value <= s.lib.pool_bytes(s.h)
        # the float weights of this model are the final Gemm's: zeroed, the output is the (zeroed) bias
        assert s.lib.dyn_maintenance(s.h, 1, s.err, 1024) == 0, s.err.value.decode()
        assert np.array_equal(s.infer(2, [x], 20), np.zeros(20, np.float32))


@pytest.mark.parametrize("model", ["MatMul_Stacked", "MatMul_Stacked2"])
def test_stacked_matmul_cases_of_the_reference(rt, model):
    """tests/cpu/TestCustomModelsFromONNX.cxx:1679-1700: Session(file, 2), infer(2, input1, input2) with the expected literals."""
    spec = em.reference_stacked_matmul_cases()[model]
    with DynamicSession(model, 2) as s:
        got = s.infer(2, spec["feeds"], 8)
    assert np.array_equal(got, np.asarray(spec["want"], np.float32))

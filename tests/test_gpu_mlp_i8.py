"""End-to-end int8 MLP (benchmark configuration 2) through the Session: bit-exact against the unfused CPU chain."""
import numpy as np
import pytest

from sofie_amd.session import Int8MLPSession
from tests import util
from tests.refmodels import int8_mlp_oracle

pytestmark = pytest.mark.gpu


def make_mlp(dims, batch, seed=1100):
    """Weights int8 U{-127..127}, input N(0,1); per-tensor symmetric scales.  The activation scales are
    calibrated once on the first 8 rows (max/127) and then frozen as model constants."""
    from oracle import binding as ob
    weights = [util.int8_sym(seed + 1 + l, dims[l] * dims[l + 1]).reshape(dims[l], dims[l + 1]) for l in range(len(dims) - 1)]
    x = util.normal(seed + 1001, batch * dims[0]).reshape(batch, dims[0])
    w_scales = [np.float32(1.0 / 127.0)] * len(weights)
    in_scales = [np.float32(np.abs(x).max() / 127.0)]
    h = x[:8]
    for l, w in enumerate(weights[:-1]):
        q = ob.quantize_linear(h, in_scales[l])
        acc = np.maximum(ob.matmul_integer(q, w, M=h.shape[0], N=w.shape[1], K=w.shape[0], omp=True), 0)
        h = ob.dequantize_linear(acc, np.float32(in_scales[l] * w_scales[l]))
        in_scales.append(np.float32(max(h.max(), 1e-6) / 127.0))
    return x, weights, w_scales, in_scales


def new_rt():
    from sofie_amd import Runtime
    return Runtime(0)


@pytest.mark.parametrize("dims,batch", [([64, 128, 96, 32], 48), ([100, 260, 130, 10], 33), ([1024, 512, 256], 256)])
def test_small_mlp_bit_exact(dims, batch):
    x, weights, w_scales, in_scales = make_mlp(dims, batch)
    rt = new_rt()
    try:
        sess = Int8MLPSession(rt, weights, w_scales, in_scales, batch)
        got = sess.infer(x)
        again = sess.infer(x)
    finally:
        rt.close()
    want = int8_mlp_oracle(x, weights, w_scales, in_scales)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got, again)
    assert (got > 0).any()


def test_config2_full_size_sampled_rows():
    """1024 -> 4096 -> 4096 -> 1024 at batch 1024: every batch row is independent, so a sample of rows is
    pushed through the CPU chain and compared bit for bit."""
    dims, batch = [1024, 4096, 4096, 1024], 1024
    x, weights, w_scales, in_scales = make_mlp(dims, batch)
    rt = new_rt()
    try:
        sess = Int8MLPSession(rt, weights, w_scales, in_scales, batch)
        got = sess.infer(x)
    finally:
        rt.close()
    rows = np.array([0, 1, 63, 64, 500, 1023, 777, 256])
    want = int8_mlp_oracle(x[rows], weights, w_scales, in_scales, omp=True)
    assert np.array_equal(got[rows].view(np.uint32), want.view(np.uint32))
    assert (got > 0).mean() > 0.2  # the network is alive: relu does not kill every unit


def test_inference_captured_in_a_hip_graph_replays_correctly():
    """infer_nosync only enqueues kernels on the context's stream (no allocation, no memset): captured once into a HIP graph
    on a caller-owned stream, every replay must reproduce the eager result, also with eager work and synchronisations in
    between and after the input buffer has been overwritten with a new batch."""
    import ctypes as C
    import torch
    from sofie_amd import Runtime
    dims, batch = [256, 512, 384, 64], 96
    x, weights, w_scales, in_scales = make_mlp(dims, batch)
    x2 = np.ascontiguousarray(x[::-1] * np.float32(0.5))
    stream = torch.cuda.Stream()
    rt = Runtime(0, external_stream=C.c_void_p(stream.cuda_stream))
    try:
        sess = Int8MLPSession(rt, weights, w_scales, in_scales, batch)
        eager, eager2 = sess.infer(x), sess.infer(x2)            # also the warm-up: kernel attributes are set outside the capture
        want = int8_mlp_oracle(x, weights, w_scales, in_scales)
        assert np.array_equal(eager.view(np.uint32), want.view(np.uint32))
        sess.upload_input(x)
        rt.sync()
        graph = torch.cuda.CUDAGraph()
        print("capturing the int8 MLP into a graph", flush=True)
        with torch.cuda.graph(graph, stream=stream):
            sess.infer_nosync()
        y = np.empty((batch, dims[-1]), dtype=np.float32)

        def fetch():
            rt.call("sofie_hip_download", y.ctypes.data_as(C.c_void_p), sess.y_ptr, C.c_size_t(y.nbytes))
            rt.sync()
            return y.copy()
        for replay, (inp, ref) in enumerate([(x, eager), (x2, eager2), (x, eager), (x, eager)]):
            sess.upload_input(inp)
            rt.call("sofie_hip_fill_zero", sess.y_ptr, C.c_size_t(y.nbytes))   # eager work between the replays
            rt.sync()
            with torch.cuda.stream(stream):   # a replay goes to torch's CURRENT stream: make that the one the download follows
                graph.replay()
            stream.synchronize()
            got = fetch()
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), "replay %d" % replay
        del graph
    finally:
        rt.close()

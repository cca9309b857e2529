#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

Workload (BASELINE config 2): int8 quantised MLP 1024 -> 4096 -> 4096 -> 1024 at batch 1024,
QuantizeLinear -> [int8 Gemm (int32 accumulate) -> Relu -> DequantizeLinear]x3, per-tensor scales,
synthetic seeded data, fp32 input already resident in HBM.  One step = one inference over the batch.
Prints ONE JSON line; `value` = inferences/s.  Also times the stand-alone int8 GEMM sweep
(M=N=K in 1024/4096/8192) and the CPU oracle on a bounded sample of batch rows.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np

INT8_PEAK = 5.0e15  # MI355X dense int8 MFMA peak, op/s
HBM_PEAK = 8.0e12


def build_mlp():
    from tests import util
    from oracle import binding as ob
    dims, batch = [1024, 4096, 4096, 1024], 1024
    weights = [util.int8_sym(1101 + l, dims[l] * dims[l + 1]).reshape(dims[l], dims[l + 1]) for l in range(3)]
    x = util.normal(2101, batch * dims[0]).reshape(batch, dims[0])
    w_scales = [np.float32(1.0 / 127.0)] * 3
    in_scales = [np.float32(np.abs(x).max() / 127.0)]
    h = x[:8]
    for l, w in enumerate(weights[:-1]):  # calibration of the frozen activation scales (model constants)
        q = ob.quantize_linear(h, in_scales[l])
        acc = np.maximum(ob.matmul_integer(q, w, M=8, N=w.shape[1], K=w.shape[0], omp=True), 0)
        h = ob.dequantize_linear(acc, np.float32(in_scales[l] * w_scales[l]))
        in_scales.append(np.float32(max(h.max(), 1e-6) / 127.0))
    return dims, batch, x, weights, w_scales, in_scales


def time_region(rt, fn, reps):
    rt.sync()
    t0 = time.perf_counter()
    rt.timer_start()
    for _ in range(reps):
        fn()
    ms = rt.timer_stop()
    wall = (time.perf_counter() - t0) * 1e3
    return ms, wall


def gemm_sweep(rt, sizes, reps=20, warmup=3):
    """Stand-alone int8 GEMM with per-channel requant + bias + relu (BASELINE config 3)."""
    from sofie_amd import runtime as R
    from tests import util
    import torch
    out = []
    for n in sizes:
        M = N = K = n
        A = util.to_dev(util.int8_sym(3001, M * K).reshape(M, K))
        Bt = util.to_dev(util.int8_sym(3002, N * K).reshape(N, K))
        bias = util.to_dev(util.int32_range(3003, N, -(1 << 15), 1 << 15))
        scale = util.to_dev(((0.5 + util.uniform01(3004, N)) / np.float32(127.0 * np.sqrt(K))).astype(np.float32))
        Y = util.dev_empty((M, N), np.int8)
        torch.cuda.synchronize()
        d = R.GemmI8Desc()
        d.M, d.N, d.K, d.transA, d.transB = M, N, K, 0, 1
        d.A, d.B, d.bias, d.scale, d.Y = util.ptr(A), util.ptr(Bt), util.ptr(bias), util.ptr(scale), util.ptr(Y)
        d.relu_out, d.out = 1, R.I8OUT_I8
        fn = lambda: rt.call("sofie_hip_gemm_i8", C.byref(d))
        for _ in range(warmup):
            fn()
        best = None
        for _ in range(3):
            ms, _ = time_region(rt, fn, reps)
            best = ms if best is None else min(best, ms)
        t = best / reps * 1e-3
        ops = 2.0 * M * N * K
        out.append({"M": M, "N": N, "K": K, "ms": round(t * 1e3, 5), "tops": round(ops / t / 1e12, 2),
                    "frac_of_int8_peak": round(ops / t / INT8_PEAK, 4),
                    "hbm_gbps_algorithmic": round((M * K + K * N + M * N + 8 * N) / t / 1e9, 1)})
        del A, Bt, Y
        torch.cuda.empty_cache()
    return out


def cpu_baseline(x, weights, w_scales, in_scales, rows):
    from oracle import binding as ob
    from tests.refmodels import int8_mlp_oracle
    threads = ob.load(True).oracle_num_threads()
    int8_mlp_oracle(x[:2], weights, w_scales, in_scales, omp=True)  # warm the caches / thread pool
    t0 = time.perf_counter()
    ref = int8_mlp_oracle(x[:rows], weights, w_scales, in_scales, omp=True)
    dt = time.perf_counter() - t0
    return ref, {"value": round(rows / dt, 2), "unit": "inferences/s", "cores": int(threads), "kind": "port",
                 "sample": "first %d of 1024 batch rows through the unfused CPU chain (oracle/sofie_oracle.c, OpenMP over rows), %.1f s"
                 % (rows, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-rows", type=int, default=64)
    ap.add_argument("--no-sweep", action="store_true", help="skip the stand-alone GEMM sweep (profiling runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg (profiling runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (the path is data-parallel over the batch; "
              "no multi-GPU figure is produced). Use --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    from sofie_amd import Runtime
    from sofie_amd.session import Int8MLPSession

    dims, batch, x, weights, w_scales, in_scales = build_mlp()
    rt = Runtime(0)
    sess = Int8MLPSession(rt, weights, w_scales, in_scales, batch)
    sess.upload_input(x)
    rt.sync()

    for _ in range(args.warmup):
        sess.infer_nosync()
    rt.sync()
    ms, wall = time_region(rt, sess.infer_nosync, args.steps)
    ms_per_step = ms / args.steps
    value = batch / (ms_per_step * 1e-3)

    # the dominant kernel alone: layers 1 and 2 (1024x4096x1024 and 1024x4096x4096) run the same kernel
    # instantiation (128x128 tiles) and hold 83% of the arithmetic; layer 3 runs the 64x64-tile one
    dom = sess.descs[:2]

    def dominant_only():
        for d in dom:
            rt.call("sofie_hip_gemm_i8", C.byref(d))
    dominant_only()
    gms, _ = time_region(rt, dominant_only, args.steps)
    launches = len(dom) * args.steps
    ops_per_inference_batch = 2.0 * batch * sum(dims[l] * dims[l + 1] for l in range(3))
    ops_per_launch = sum(2.0 * d.M * d.N * d.K for d in dom) / len(dom)
    avg_launch_s = gms * 1e-3 / launches
    achieved = ops_per_launch / avg_launch_s

    # what the matrix cores of this board sustain with no memory traffic (constant / toggling operands)
    import torch
    scratch = torch.empty(1 << 20, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    probe = {}
    for name, rnd in (("constant_operands", 0), ("random_operands", 1)):
        v = C.c_double()
        rt.call("sofie_hip_mfma_i8_probe", C.c_void_p(scratch.data_ptr()), C.c_size_t(scratch.numel() * 4), 20000, rnd, C.byref(v))
        probe[name] = round(v.value / 1e12, 1)

    # parity of what was timed, against the oracle on the sampled rows
    y = np.empty((batch, dims[-1]), dtype=np.float32)
    rt.call("sofie_hip_download", y.ctypes.data_as(C.c_void_p), sess.y_ptr, C.c_size_t(y.nbytes))
    rt.sync()
    if args.no_cpu:
        cpu, parity = None, None
    else:
        ref, cpu = cpu_baseline(x, weights, w_scales, in_scales, args.cpu_rows)
        parity = bool(np.array_equal(y[:args.cpu_rows].view(np.uint32), ref.view(np.uint32)))

    sweep = [] if args.no_sweep else gemm_sweep(rt, [1024, 4096, 8192])
    rt.close()

    algo_bytes = sum(w.size for w in weights) + 4 * batch * dims[0] + 4 * batch * dims[-1]
    line = {
        "metric": "inferences/sec @batch 1024 int8 MLP; int8 GEMM TOPS & % of MI355X MFMA peak",
        "value": round(value, 1), "unit": "inferences/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "int8 MLP 1024->4096->4096->1024, batch 1024, Q -> [i8 Gemm(i32) -> Relu -> DQ]x3, "
                               "per-tensor symmetric scales, input resident in HBM (BASELINE configs[1])",
                   "global_batch": batch, "launches_per_step": 4, "wall_ms_per_step": round(wall / args.steps, 5),
                   "parity_vs_oracle_rows": args.cpu_rows, "parity_bit_exact": parity,
                   "mlp_tops": round(ops_per_inference_batch / (ms_per_step * 1e-3) / 1e12, 2),
                   "mlp_algorithmic_bytes": algo_bytes,
                   "int8_mfma_register_only_tops": probe,
                   "gemm_sweep_int8_requant_bias_relu": sweep},
        "roofline": {"bound": "mfma", "achieved": round(achieved / 1e12, 2), "peak": INT8_PEAK / 1e12, "unit": "TFLOP/s",
                     "frac": round(achieved / INT8_PEAK, 4), "traffic": None,
                     "frac_of_sustained_random_operand_rate": round(achieved / 1e12 / probe["random_operands"], 4),
                     "kernel": "mfma8_gemm_dma_kernel<MfmaI8, 128, 128, ...> (layers 1 and 2 of the MLP: 2 launches per inference, "
                               "avg %.2f us, %.3e int8 op per launch on average)" % (avg_launch_s * 1e6, ops_per_launch)},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

"""The benchmark's Sessions: the generator emits each benchmark model at its full size (weights in a safetensors file) and a
small harness is compiled around the emitted header, the way the reference's benchmark compiles one around its generated
code (benchmark/src/BenchmarkEmitter.cxx.in:486-504).  build_bench_models() runs at build time on the CPU; the benchmark and
the full-size parity tests only load the libraries."""
import os
import subprocess

import numpy as np

from sofie_amd.benchsupport import models
from sofie_amd.benchsupport import onnx_write as ow

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
OUT = os.path.join(ROOT, "sofie_amd", "benchsupport", "emitted")
EMIT = os.path.join(ROOT, "sofie_amd", "emit", "bin", "sofie_hip_emit")

BENCH_HARNESS = r'''
#include "%(model)s_GPU_HIP.hxx"
#include <chrono>
#include <cstring>
using Session = SOFIE_%(model)s::Session;
static void set_error(char *err, int errlen, const char *what)
{
   std::strncpy(err, what, errlen - 1);
   err[errlen - 1] = 0;
}
extern "C" void *bench_open(const char *weights, char *err, int errlen)
{
   try {
      return new Session(weights);
   } catch (const std::exception &e) {
      set_error(err, errlen, e.what());
      return nullptr;
   }
}
extern "C" void bench_close(void *h) { delete static_cast<Session *>(h); }
// uploads one batch into the Session's input region; returns 0, or 1 with the exception text in err
extern "C" int bench_upload(void *h, const void *x, unsigned long nbytes, char *err, int errlen)
{
   try {
      Session &s = *static_cast<Session *>(h);
      if (sofie_hip_upload(s.context(), s.device_input_%(input)s(), x, nbytes) || sofie_hip_sync(s.context()))
         throw std::runtime_error(sofie_hip_last_error());
      return 0;
   } catch (const std::exception &e) {
      set_error(err, errlen, e.what());
      return 1;
   }
}
extern "C" int bench_download(void *h, void *y, unsigned long nbytes, char *err, int errlen)
{
   try {
      Session &s = *static_cast<Session *>(h);
      if (sofie_hip_download(s.context(), y, s.device_output_%(output)s(), nbytes) || sofie_hip_sync(s.context()))
         throw std::runtime_error(sofie_hip_last_error());
      return 0;
   } catch (const std::exception &e) {
      set_error(err, errlen, e.what());
      return 1;
   }
}
// `steps` inferences enqueued back to back, one wait: wall-clock milliseconds of the region (and, through *event_ms, what a pair
// of events on the Session's stream measured); negative on failure
extern "C" double bench_run(void *h, int steps, float *event_ms, char *err, int errlen)
{
   try {
      Session &s = *static_cast<Session *>(h);
      s.sync();
      const auto t0 = std::chrono::steady_clock::now();
      if (sofie_hip_timer_start(s.context()))
         throw std::runtime_error(sofie_hip_last_error());
      for (int i = 0; i < steps; ++i)
         s.infer_nosync();
      float ms = 0;
      if (sofie_hip_timer_stop(s.context(), &ms)) // records the second event and waits for it
         throw std::runtime_error(sofie_hip_last_error());
      const auto t1 = std::chrono::steady_clock::now();
      if (event_ms)
         *event_ms = ms;
      return std::chrono::duration<double, std::milli>(t1 - t0).count();
   } catch (const std::exception &e) {
      set_error(err, errlen, e.what());
      return -1.0;
   }
}
'''




def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), r.stdout))
    return r.stdout


def compile_shared(src, lib, include_dir):
    _run(["g++", "-O1", "-std=c++20", "-fPIC", "-shared", "-I" + os.path.join(ROOT, "include"), "-I" + include_dir, src, "-o", lib,
          "-L" + os.path.join(ROOT, "sofie_amd", "lib"), "-lsofie_hip", "-Wl,-rpath," + os.path.join(ROOT, "sofie_amd", "lib"),
          "-Wl,-rpath,$ORIGIN/../../lib"])
    return lib


BENCH_MODEL = "Config2_int8_MLP"
CNN_MODEL = "Config5_int8_CNN"
GEMM_MODEL = "Config3_int8_GEMM_8192"


def bench_mlp_spec():
    """benchmark configuration 2 at its full size: 1024 -> 4096 -> 4096 -> 1024, batch 1024."""
    return models.int8_mlp([1024, 4096, 4096, 1024], 1024, seed=1100)


def bench_cnn_spec():
    """benchmark configuration 5 at its full size: batch 256, 64 x 64 images."""
    return models.int8_cnn(256, 64)


def bench_gemm_spec():
    """benchmark configuration 3 at M = N = K = 8192 as a one-operator model."""
    return models.int8_gemm_requant(8192)


BENCH_SPECS = {BENCH_MODEL: bench_mlp_spec, CNN_MODEL: bench_cnn_spec, GEMM_MODEL: bench_gemm_spec}


def build_bench_model(model, keep_onnx=False):
    """Emits one benchmark model at full size with its weights in a safetensors file and compiles the benchmark harness
    around the emitted Session.  The ONNX file is an intermediate (the weights travel in the safetensors file)."""
    os.makedirs(OUT, exist_ok=True)
    spec = BENCH_SPECS[model]()
    p = os.path.join(OUT, model + ".onnx")
    ow.write(p, spec["nodes"], spec["inputs"], spec["outputs"], spec["init"], name=model)
    _run([EMIT, p, OUT, "--safetensors"])
    if not keep_onnx:
        os.remove(p)
    src = os.path.join(OUT, model + "_bench.cxx")
    with open(src, "w") as f:
        f.write(BENCH_HARNESS % dict(model=model, input=spec["inputs"][0][0], output=spec["outputs"][0][0]))
    return compile_shared(src, os.path.join(OUT, "lib%s_bench.so" % model), OUT)


def build_bench_models():
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=3) as ex:
        return list(ex.map(build_bench_model, BENCH_SPECS))


class BenchSession:
    """An emitted Session of a full-size benchmark model behind its benchmark harness (ctypes)."""

    def __init__(self, model=BENCH_MODEL):
        import ctypes as C
        lib_path = os.path.join(OUT, "lib%s_bench.so" % model)
        if not os.path.exists(lib_path):
            raise RuntimeError("%s is missing: __graft_entry__.build() emits and compiles it" % lib_path)
        self.C = C
        self.lib = C.CDLL(lib_path)
        self.lib.bench_open.restype = C.c_void_p
        self.lib.bench_open.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
        self.lib.bench_close.argtypes = [C.c_void_p]
        self.lib.bench_upload.argtypes = [C.c_void_p, C.c_void_p, C.c_ulong, C.c_char_p, C.c_int]
        self.lib.bench_download.argtypes = [C.c_void_p, C.c_void_p, C.c_ulong, C.c_char_p, C.c_int]
        self.lib.bench_run.restype = C.c_double
        self.lib.bench_run.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_float), C.c_char_p, C.c_int]
        self.err = C.create_string_buffer(1024)
        self.h = self.lib.bench_open(os.path.join(OUT, model + "_GPU_HIP.safetensors").encode(), self.err, 1024)
        if not self.h:
            raise RuntimeError("emitted Session: " + self.err.value.decode())

    def close(self):
        if self.h:
            self.lib.bench_close(self.h)
            self.h = None

    def upload(self, x):
        """One batch into the Session's input region (the array's own element type)."""
        x = np.ascontiguousarray(x)
        if self.lib.bench_upload(self.h, x.ctypes.data, x.nbytes, self.err, 1024):
            raise RuntimeError(self.err.value.decode())

    def download(self, shape, dtype=np.float32):
        y = np.empty(shape, dtype=dtype)
        if self.lib.bench_download(self.h, y.ctypes.data, y.nbytes, self.err, 1024):
            raise RuntimeError(self.err.value.decode())
        return y

    def run(self, steps):
        """steps x infer_nosync + one wait: (wall ms, event ms) of the region."""
        ev = self.C.c_float()
        wall = self.lib.bench_run(self.h, steps, self.C.byref(ev), self.err, 1024)
        if wall < 0:
            raise RuntimeError(self.err.value.decode())
        return wall, ev.value

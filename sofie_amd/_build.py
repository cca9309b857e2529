"""Build steps: hipcc for the gfx950 runtime library, make for the CPU oracle (the checker)."""
import os
import shutil
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "sofie_amd", "csrc")
LIB_DIR = os.path.join(ROOT, "sofie_amd", "lib")
LIB = os.path.join(LIB_DIR, "libsofie_hip.so")

HIP_SOURCES = ["runtime.hip", "gemm_i8.hip", "gemm_f32.hip", "gemm_fp8.hip", "conv_i8.hip", "eltwise.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-fast-math", "-ffp-contract=off",
    "-Wall", "-Wno-unused-function", "-Wno-pass-failed",
]


def _hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def _run(cmd, cwd=None):
    print("+", " ".join(cmd), flush=True)
    r = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if r.returncode != 0:
        raise RuntimeError("command failed (%d): %s" % (r.returncode, " ".join(cmd)))


def build_hip_library(jobs=8):
    """Compiles every HIP source for gfx950 and links sofie_amd/lib/libsofie_hip.so."""
    from concurrent.futures import ThreadPoolExecutor
    lib_dir = LIB_DIR
    lib = LIB
    os.makedirs(lib_dir, exist_ok=True)
    obj_dir = os.path.join(ROOT, "build", "obj")
    os.makedirs(obj_dir, exist_ok=True)
    flags = HIPCC_FLAGS
    hipcc = _hipcc()
    sources = [s for s in HIP_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(obj_dir, s.replace(".hip", ".o")) for s in sources]

    def compile_one(pair):
        src, obj = pair
        _run([hipcc] + flags + ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(compile_one, zip(sources, objs)))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    return lib


def build_oracle():
    """Builds the CPU checker (and oracle/_ref when the reference checkout is present)."""
    _run(["make", "-B", "-C", os.path.join(ROOT, "oracle"), "all"])


def build_all():
    lib = build_hip_library()
    build_oracle()
    _run(["make", "-C", os.path.join(ROOT, "sofie_amd", "emit"), "-B", "-j8", "all"])
    return lib


if __name__ == "__main__":
    build_all()
    sys.exit(0)

"""sofie_amd: gfx950 (MI355X) runtime and code-emission backend for SOFIE's Gemm / Conv hot path.

The product is the C-ABI library built from ``sofie_amd/csrc`` (declared in ``include/sofie_hip.h``)
and the C++ emitter under ``sofie_amd/emit``.  This Python package is only the thin loader that the
tests and the benchmark use to reach the C-ABI; it holds no compute and no CPU fallback.
"""
from .runtime import Runtime, SofieHipError, lib_path, load_library  # noqa: F401

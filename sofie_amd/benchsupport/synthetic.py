"""Shared helpers of the benchmark and the tests: a counter-based generator that rebuilds the same
synthetic tensors anywhere (SplitMix64 of (seed, index)), and torch-backed device buffers whose raw
pointers are handed to the C-ABI."""
import ctypes as C

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(seed, n, offset=0):
    """n 64-bit values: splitmix64 finaliser of (seed * golden + index)."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset, offset + n, dtype=np.uint64)
        z = (idx + np.uint64(seed) * np.uint64(0x9E3779B97F4A7C15)) + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return z


def uniform01(seed, n):
    """U[0,1) with 24 random bits, exactly representable in fp32."""
    return ((splitmix64(seed, n) >> np.uint64(40)).astype(np.float32) * np.float32(1.0 / (1 << 24))).astype(np.float32)


def normal(seed, n, sigma=1.0):
    """N(0, sigma) by Box-Muller in float64, rounded to fp32."""
    m = (n + 1) // 2
    u = splitmix64(seed, 2 * m)
    u1 = ((u[:m] >> np.uint64(11)).astype(np.float64) + 1.0) / float(1 << 53)
    u2 = (u[m:] >> np.uint64(11)).astype(np.float64) / float(1 << 53)
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.concatenate([r * np.cos(2 * np.pi * u2), r * np.sin(2 * np.pi * u2)])[:n]
    return (out * sigma).astype(np.float32)


def int8_sym(seed, n):
    """int8 uniform on {-127..127}."""
    return ((splitmix64(seed, n) >> np.uint64(33)) % np.uint64(255)).astype(np.int64).astype(np.int16).__sub__(127).astype(np.int8)


def int32_range(seed, n, lo, hi):
    span = np.uint64(hi - lo + 1)
    return ((splitmix64(seed, n) >> np.uint64(20)) % span).astype(np.int64).__add__(lo).astype(np.int32)


# ---- device buffers (torch is only the allocator) ---------------------------------------------------------

def to_dev(a):
    import torch
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t.cuda()


def dev_empty(shape, dtype):
    import torch
    tdt = {np.int8: torch.int8, np.uint8: torch.uint8, np.int32: torch.int32, np.float32: torch.float32,
           np.uint16: torch.int16}[np.dtype(dtype).type]
    return torch.empty(shape, dtype=tdt, device="cuda")


def ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def to_host(t, dtype=None):
    import torch
    torch.cuda.synchronize()
    a = t.cpu().numpy()
    if dtype is not None:
        a = a.view(dtype)
    return a

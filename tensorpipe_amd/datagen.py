"""Seeded synthetic payloads (numpy views over the C generator in csrc/datagen)."""
import numpy as np

from . import _native


def uniform_u8(seed, nbytes):
    out = np.empty(nbytes, dtype=np.uint8)
    _native.datagen().tpdg_fill_u8(seed, out.ctypes.data, nbytes)
    return out


def normal(seed, n_elems, dtype, sigma=1.0):
    """N(0, sigma) stored as 'f32', 'bf16' or 'f16'; bf16/f16 come back as raw uint16."""
    lib = _native.datagen()
    if dtype == "f32":
        out = np.empty(n_elems, dtype=np.float32)
        lib.tpdg_fill_normal_f32(seed, float(sigma), out.ctypes.data, n_elems)
    elif dtype == "bf16":
        out = np.empty(n_elems, dtype=np.uint16)
        lib.tpdg_fill_normal_bf16(seed, float(sigma), out.ctypes.data, n_elems)
    elif dtype == "f16":
        out = np.empty(n_elems, dtype=np.uint16)
        lib.tpdg_fill_normal_f16(seed, float(sigma), out.ctypes.data, n_elems)
    else:
        raise ValueError(dtype)
    return out


def loguniform_sizes(seed, lo, hi, n):
    out = np.empty(n, dtype=np.uint64)
    _native.datagen().tpdg_loguniform_sizes(seed, lo, hi, out.ctypes.data, n)
    return out


def bench_pattern(nbytes):
    out = np.empty(nbytes, dtype=np.uint8)
    _native.datagen().tpdg_bench_pattern(out.ctypes.data, nbytes)
    return out


def fnv1a64(arr):
    a = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
    return int(_native.datagen().tpdg_fnv1a64(a.ctypes.data, a.size))


# Seeds of the benchmark configurations (config k uses SEED_BASE + k).
SEED_BASE = 0x7E500000

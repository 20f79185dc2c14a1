"""Counter-based synthetic inputs for tests and the benchmark (the reference has no seeded RNG; `uniform()` there draws
from `rand::rng()`, core/tensor.rs:787-807).  Element i of tensor `stream` under `seed` is a pure function of
(seed, stream, i): the numpy code here and the device kernel in csrc/rt_datagen.hip produce identical bits."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_M = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)).astype(np.uint64)
        z = x
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _key(seed: int, stream: int) -> np.uint64:
    with np.errstate(over="ignore"):
        a = _splitmix64(np.array([seed], dtype=np.uint64))[0]
        b = np.uint64((stream * 0xD1342543DE82EF95) & 0xFFFFFFFFFFFFFFFF)
        return _splitmix64(np.array([a ^ b], dtype=np.uint64))[0]


def _draw(key, idx: np.ndarray, k: int) -> np.ndarray:
    with np.errstate(over="ignore"):
        return _splitmix64(key + idx * np.uint64(8) + np.uint64(k))


def _irwin_hall(key, idx):
    s = np.zeros(idx.shape, dtype=np.int64)
    for k in range(6):
        r = _draw(key, idx, k)
        s += (r >> np.uint64(40)).astype(np.int64) + ((r >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.int64)
    return s - 6 * (1 << 24)


def uniform(dtype, n: int, seed: int, stream: int, start: int = 0) -> np.ndarray:
    """U[-1, 1) as f32 or f64, elements start .. start+n of the stream."""
    idx = np.arange(start, start + n, dtype=np.uint64)
    r = _draw(_key(seed, stream), idx, 0)
    if np.dtype(dtype) == np.float32:
        return ((r >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -23) - np.float32(1.0)).astype(np.float32)
    return (r >> np.uint64(11)).astype(np.float64) * 2.0 ** -52 - 1.0


def normal(dtype, n: int, seed: int, stream: int, sigma: float = 1.0, start: int = 0) -> np.ndarray:
    """Approximately N(0, sigma): Irwin-Hall sum of twelve 24-bit uniforms."""
    idx = np.arange(start, start + n, dtype=np.uint64)
    s = _irwin_hall(_key(seed, stream), idx)
    if np.dtype(dtype) == np.float32:
        return (s.astype(np.float32) * np.float32(sigma * 2.0 ** -24)).astype(np.float32)
    return s.astype(np.float64) * (sigma * 2.0 ** -24)


def integers(n: int, seed: int, stream: int, lo: int, hi: int, start: int = 0) -> np.ndarray:
    """i32 uniform in [lo, hi]."""
    idx = np.arange(start, start + n, dtype=np.uint64)
    r = _draw(_key(seed, stream), idx, 0)
    return (np.int64(lo) + (r % np.uint64(hi - lo + 1)).astype(np.int64)).astype(np.int32)


# ---- device-side generation (same bits, no PCIe transfer) ---------------------------------------------------------------
_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "librt_datagen.so")
_lib = None


def _dev():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise ImportError(f"{_LIB} is missing: build it with `python -m rtensors_amd.build`")
        _lib = C.CDLL(_LIB)
        _lib.rtd_generate.restype = C.c_int32
        _lib.rtd_generate.argtypes = [C.c_int32, C.c_int32, C.c_uint64, C.c_uint64, C.c_double, C.c_double, C.c_void_p, C.c_uint64]
    return _lib


def fill_device(buf, dist: str, seed: int, stream: int, p0: float = 1.0, p1: float = 0.0) -> None:
    """Fill a HipBuf (f32 / f64 / i32) on the device.  dist: 'uniform' | 'normal' (sigma=p0) | 'int' ([p0, p1])."""
    code = {"uniform": 0, "normal": 1, "int": 2}[dist]
    buf.backend.sync()
    rc = _dev().rtd_generate(buf.dtype, code, seed, stream, float(p0), float(p1), buf.ptr, buf.len)
    if rc != 0:
        raise RuntimeError(f"rtd_generate failed with code {rc}")

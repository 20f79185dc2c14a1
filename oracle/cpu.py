"""TEST INFRASTRUCTURE ONLY -- never imported by the product path.

ctypes front end of oracle/_build/librt_oracle.so (the C++ restatement of the reference `Cpu` backend,
oracle/cpu_oracle.cpp).  Buffers are 1-D numpy arrays; layouts are `oracle.meta.MetaTensor`.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

import numpy as np

from .meta import MetaTensor, TensorError

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "librt_oracle.so")

# dtype codes: core/value.rs:567-581
U8, I8, U16, I16, U32, U128, I32, U64, I64, I128, F32, F64, BOOL = range(13)

# 128-bit integers have no numpy scalar type; they travel as 16 raw little-endian bytes.
V16 = np.dtype("V16")

NP_DTYPE = {
    U8: np.dtype(np.uint8), I8: np.dtype(np.int8), U16: np.dtype(np.uint16), I16: np.dtype(np.int16),
    U32: np.dtype(np.uint32), I32: np.dtype(np.int32), U64: np.dtype(np.uint64), I64: np.dtype(np.int64),
    F32: np.dtype(np.float32), F64: np.dtype(np.float64), BOOL: np.dtype(np.bool_), U128: V16, I128: V16,
}
DTYPE_NAME = {U8: "u8", I8: "i8", U16: "u16", I16: "i16", U32: "u32", U128: "u128", I32: "i32", U64: "u64",
              I64: "i64", I128: "i128", F32: "f32", F64: "f64", BOOL: "bool"}
DTYPE_BY_NAME = {v: k for k, v in DTYPE_NAME.items()}

# op codes (see oracle/cpu_oracle.cpp for the reference lines)
UNARY = {n: i for i, n in enumerate(
    "neg relu sigmoid silu tanh abs sqrt ln expm1 ln1p floor ceil round trunc sin cos tan asin acos atan sinh cosh "
    "asinh acosh atanh rsqrt reciprocal square cube exp sign".split())}
SCALAR = {n: i for i, n in enumerate("add sub mul div log log1p leaky_relu elu leaky_grad".split())}
BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3}
REDUCE = {"sum": 1, "prod": 2, "max": 3, "min": 4, "mean": 5,
          # the Cuda backend's other kinds (ops/reduction/mod.rs:161-175; payload of Variance / Stdev / Norm in the flag bits)
          "pop_var": 6, "var": 6 | 0x100, "pop_std": 6 | 0x200, "std": 6 | 0x300, "logsumexp": 7, "l1_norm": 8 | 0x100, "l2_norm": 8 | 0x200,
          "argmax": 9, "argmin": 10}
STAT_OPS = ("pop_var", "var", "pop_std", "std", "logsumexp", "l1_norm", "l2_norm")
ARG_OPS = ("argmax", "argmin")

_ERR = {1: "UnsupportedOperation", 2: "IdxOutOfBounds(panic)", 3: "ArithmeticPanic", 4: "WrongDims", 5: "UnsupportedOp"}


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile (g++ only)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "cpu_oracle.cpp")):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        sz, i64p, szp, vp, ip = C.c_size_t, C.POINTER(C.c_int64), C.POINTER(C.c_size_t), C.c_void_p, C.POINTER(C.c_int)
        i64 = C.c_int64
        L.orc_dtype_size.argtypes = [C.c_int]
        L.orc_is_contiguous.argtypes = [sz, C.c_int, szp, i64p]
        L.orc_unary.argtypes = [C.c_int, C.c_int, vp, sz, sz, C.c_int, szp, i64p, ip]
        L.orc_scalar.argtypes = [C.c_int, C.c_int, vp, sz, vp, sz, C.c_int, szp, i64p, ip]
        L.orc_fill.argtypes = [C.c_int, vp, sz, vp, sz, C.c_int, szp, i64p, ip]
        L.orc_broadcast.argtypes = [C.c_int, C.c_int, C.c_int, szp,
                                    vp, sz, sz, i64p, vp, sz, sz, i64p, vp, sz, sz, i64p]
        L.orc_reduce_flat.argtypes = [C.c_int, C.c_int, vp, sz, vp, sz, sz, sz]
        L.orc_reduce_nd.argtypes = [C.c_int, C.c_int, vp, sz, sz, C.c_int, szp, i64p, vp, sz, C.c_int, C.c_int]
        L.orc_gather.argtypes = [C.c_int, vp, sz, sz, C.c_int, szp, i64p, vp, sz]
        L.orc_reduce_stat.argtypes = [C.c_int, C.c_int, vp, sz, sz, sz, sz, sz, vp, sz]
        L.orc_argmax.argtypes = [C.c_int, C.c_int, vp, sz, sz, sz, sz, sz, vp, sz]
        L.orc_equal.argtypes = [C.c_int, vp, vp, sz]
        L.orc_matmul.argtypes = [C.c_int, vp, sz, sz, i64, i64, i64, vp, sz, sz, i64, i64, i64, vp, sz, sz, sz, sz, sz]
        _lib = L
    return _lib


def _check(rc: int, what: str):
    if rc != 0:
        raise TensorError(_ERR.get(rc, f"code{rc}"), what)


def _shape_arr(shape):
    return (C.c_size_t * max(len(shape), 1))(*shape)


def _stride_arr(strides):
    return (C.c_int64 * max(len(strides), 1))(*strides)


def _ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"] and a.ndim == 1
    return a.ctypes.data_as(C.c_void_p)


def value_bytes(dtype: int, value) -> np.ndarray:
    """One element of `dtype` as a 1-element numpy array (python ints for the 128-bit types)."""
    if dtype in (U128, I128):
        v = int(value) & ((1 << 128) - 1)
        return np.frombuffer(v.to_bytes(16, "little"), dtype=V16).copy()
    return np.array([value], dtype=NP_DTYPE[dtype])


def from_ints(dtype: int, values) -> np.ndarray:
    """Build a buffer from python numbers (needed for the 128-bit dtypes)."""
    if dtype in (U128, I128):
        raw = b"".join((int(v) & ((1 << 128) - 1)).to_bytes(16, "little") for v in values)
        return np.frombuffer(raw, dtype=V16).copy()
    return np.array(list(values), dtype=NP_DTYPE[dtype])


def to_ints(dtype: int, buf: np.ndarray):
    if dtype in (U128, I128):
        out = []
        raw = buf.tobytes()
        for i in range(0, buf.size * 16, 16):
            v = int.from_bytes(raw[i:i + 16], "little")
            if dtype == I128 and v >= 1 << 127:
                v -= 1 << 128
            out.append(v)
        return out
    return buf.tolist()


def unary(dtype: int, op: str, buf: np.ndarray, meta: MetaTensor) -> str:
    """`Backend::apply_<op>` incl. the three-way layout dispatch; returns the loop that ran."""
    path = C.c_int(-1)
    rc = lib().orc_unary(dtype, UNARY[op], _ptr(buf), buf.size, meta.offset, meta.rank(), _shape_arr(meta.shape),
                         _stride_arr(meta.strides), C.byref(path))
    _check(rc, f"apply_{op}")
    return ("contiguous", "1d_strided", "nd")[path.value]


def scalar(dtype: int, op: str, buf: np.ndarray, value, meta: MetaTensor) -> str:
    """`Backend::scalar_apply_<op>`."""
    path = C.c_int(-1)
    v = value_bytes(dtype, value)
    rc = lib().orc_scalar(dtype, SCALAR[op], _ptr(buf), buf.size, _ptr(v), meta.offset, meta.rank(),
                          _shape_arr(meta.shape), _stride_arr(meta.strides), C.byref(path))
    _check(rc, f"scalar_apply_{op}")
    return ("contiguous", "1d_strided", "nd")[path.value]


def fill(dtype: int, buf: np.ndarray, value, meta: MetaTensor) -> str:
    """`Backend::fill`."""
    path = C.c_int(-1)
    v = value_bytes(dtype, value)
    rc = lib().orc_fill(dtype, _ptr(buf), buf.size, _ptr(v), meta.offset, meta.rank(), _shape_arr(meta.shape),
                        _stride_arr(meta.strides), C.byref(path))
    _check(rc, "fill")
    return ("contiguous", "1d_strided", "nd")[path.value]


def broadcast(dtype: int, op: str, left: np.ndarray, lmeta: MetaTensor, right: np.ndarray, rmeta: MetaTensor,
              dst: np.ndarray, dmeta: MetaTensor) -> None:
    """`Backend::broadcast`; operands arrive pre-broadcast (equal shapes, expansion as stride 0); dst may be left."""
    assert lmeta.shape == rmeta.shape == dmeta.shape
    rc = lib().orc_broadcast(dtype, BINARY[op], dmeta.rank(), _shape_arr(dmeta.shape),
                             _ptr(left), left.size, lmeta.offset, _stride_arr(lmeta.strides),
                             _ptr(right), right.size, rmeta.offset, _stride_arr(rmeta.strides),
                             _ptr(dst), dst.size, dmeta.offset, _stride_arr(dmeta.strides))
    _check(rc, f"broadcast {op}")


def reduce_flat(dtype: int, op: str, src: np.ndarray, start: int, length: int) -> np.ndarray:
    """`Backend::apply_reduce_contiguous_flat` -> 1-element buffer."""
    dst = np.zeros(1, dtype=NP_DTYPE[dtype])
    rc = lib().orc_reduce_flat(dtype, REDUCE[op], _ptr(src), src.size, _ptr(dst), dst.size, start, length)
    _check(rc, f"reduce_flat {op}")
    return dst


def reduce_nd(dtype: int, op: str, src: np.ndarray, meta: MetaTensor, dim: int, honour_offset: bool = True,
              dst: Optional[np.ndarray] = None) -> np.ndarray:
    """`Backend::apply_reduce_contiguous_nd`; `honour_offset=False` is the literal Cpu behaviour (offset ignored)."""
    outputs = meta.outer_dimensions(dim) * meta.inner_dimensions(dim)
    if dst is None:
        dst = np.zeros(outputs, dtype=NP_DTYPE[dtype])
    rc = lib().orc_reduce_nd(dtype, REDUCE[op], _ptr(src), src.size, meta.offset, meta.rank(), _shape_arr(meta.shape),
                             _stride_arr(meta.strides), _ptr(dst), dst.size, dim, 1 if honour_offset else 0)
    _check(rc, f"reduce_nd {op}")
    return dst


def _outer_r_inner(meta: MetaTensor, dim: Optional[int]):
    """(outer, R, inner) of a contiguous view reduced over `dim` (None: everything, the flat form)."""
    if dim is None:
        return 1, meta.size(), 1
    if not meta.is_contiguous():
        raise TensorError("WrongDims", "Reduction over non-contiguous tensors is not implemented yet.")
    return meta.outer_dimensions(dim), meta.shape[dim], meta.inner_dimensions(dim)


def reduce_stat(dtype: int, op: str, src: np.ndarray, meta: MetaTensor, dim: Optional[int]) -> np.ndarray:
    """Variance / stdev / logsumexp / norms over `dim` (None: the whole contiguous view): the per-element rules of the reference's Cuda
    kernels applied in index order (oracle/cpu_oracle.cpp)."""
    outer, r, inner = _outer_r_inner(meta, dim)
    dst = np.zeros(max(outer * inner, 1), dtype=NP_DTYPE[dtype])
    rc = lib().orc_reduce_stat(dtype, REDUCE[op], _ptr(src), src.size, meta.offset, outer, r, inner, _ptr(dst), dst.size)
    _check(rc, f"reduce {op}")
    return dst[:outer * inner]


def argmax(dtype: int, op: str, src: np.ndarray, meta: MetaTensor, dim: Optional[int]) -> np.ndarray:
    """`apply_argmax_contiguous_flat` / `_nd`: u64 index of the first extremum along `dim` (None: inside the whole view)."""
    outer, r, inner = _outer_r_inner(meta, dim)
    dst = np.zeros(max(outer * inner, 1), dtype=np.uint64)
    rc = lib().orc_argmax(dtype, REDUCE[op], _ptr(src), src.size, meta.offset, outer, r, inner, _ptr(dst), dst.size)
    _check(rc, op)
    return dst[:outer * inner]


def gather(dtype: int, src: np.ndarray, meta: MetaTensor) -> np.ndarray:
    """`view_to_contiguous` (core/tensor.rs:299-325): row-major copy of the elements a view addresses."""
    dst = np.zeros(meta.size(), dtype=NP_DTYPE[dtype])
    rc = lib().orc_gather(dtype, _ptr(src), src.size, meta.offset, meta.rank(), _shape_arr(meta.shape),
                          _stride_arr(meta.strides), _ptr(dst), dst.size)
    _check(rc, "gather")
    return dst


def matmul(dtype: int, lhs: np.ndarray, lhs_meta: MetaTensor, rhs: np.ndarray, rhs_meta: MetaTensor, b: int, m: int, k: int, n: int) -> np.ndarray:
    """`BackendMatMul::matmul` of the Cpu backend (backend/cpu.rs:725-951): dst[batch] = lhs[batch] @ rhs[batch], dst row-major.
    The batch stride is `strides[rank - 3]` (0 for rank 2), rows / columns step by the last two strides."""
    def parts(meta):
        r = meta.rank()
        return meta.offset, meta.strides[r - 2], meta.strides[r - 1], (meta.strides[r - 3] if r > 2 else 0)
    lo, lrs, lcs, lbs = parts(lhs_meta)
    ro, rrs, rcs, rbs = parts(rhs_meta)
    dst = np.zeros(b * m * n, dtype=NP_DTYPE[dtype])
    rc = lib().orc_matmul(dtype, _ptr(lhs), lhs.size, lo, lrs, lcs, lbs, _ptr(rhs), rhs.size, ro, rrs, rcs, rbs, _ptr(dst), dst.size, b, m, k, n)
    _check(rc, "matmul")
    return dst


def equal(dtype: int, a: np.ndarray, b: np.ndarray) -> bool:
    """`Box<[T]> == Box<[T]>`: lengths equal and every pair `==` (NaN != NaN, -0.0 == 0.0)."""
    if a.size != b.size:
        return False
    return bool(lib().orc_equal(dtype, _ptr(a), _ptr(b), a.size))

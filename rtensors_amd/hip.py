"""`Hip`: host-side mirror of the reference's `Backend` trait (libs/rtensors/src/backend/mod.rs:216-472) over the
C ABI.  Method names, argument meaning and error behaviour follow the trait; buffers are `HipBuf` (device pointer +
length + dtype, the counterpart of `CudaBuf`, backend/cuda.rs:53-57).  Host data crosses as 1-D numpy arrays."""
from __future__ import annotations

import ctypes as C
from typing import Sequence, Tuple

import numpy as np

from . import _ffi
from ._ffi import lib

# dtype codes: core/value.rs:567-581
U8, I8, U16, I16, U32, U128, I32, U64, I64, I128, F32, F64, BOOL = range(13)
V16 = np.dtype("V16")
NP_DTYPE = {
    U8: np.dtype(np.uint8), I8: np.dtype(np.int8), U16: np.dtype(np.uint16), I16: np.dtype(np.int16),
    U32: np.dtype(np.uint32), I32: np.dtype(np.int32), U64: np.dtype(np.uint64), I64: np.dtype(np.int64),
    F32: np.dtype(np.float32), F64: np.dtype(np.float64), BOOL: np.dtype(np.bool_), U128: V16, I128: V16,
}
DTYPE_BY_NAME = {"u8": U8, "i8": I8, "u16": U16, "i16": I16, "u32": U32, "u128": U128, "i32": I32, "u64": U64, "i64": I64,
                 "i128": I128, "f32": F32, "f64": F64, "bool": BOOL}

UNARY = {n: i for i, n in enumerate(
    "neg relu sigmoid silu tanh abs sqrt ln expm1 ln1p floor ceil round trunc sin cos tan asin acos atan sinh cosh "
    "asinh acosh atanh rsqrt reciprocal square cube exp sign step abs_grad".split())}
SCALAR = {n: i for i, n in enumerate("add sub mul div log log1p leaky_relu elu leaky_grad".split())}
CONTIGUITY = {"row_major": 0, "column_major": 1, "none": 2}     # core/meta.rs:744-750
BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3}
# ReductionOpTypes::get_code (ops/reduction/mod.rs:161-175) in the low byte; the payload of Variance / Stdev / Norm in the flag bits
REDUCE = {"sum": 1, "prod": 2, "max": 3, "min": 4, "mean": 5,
          "pop_var": 6, "var": 6 | 0x100, "pop_std": 6 | 0x200, "std": 6 | 0x300, "logsumexp": 7, "l1_norm": 8 | 0x100, "l2_norm": 8 | 0x200,
          "argmax": 9, "argmin": 10}

# rt_status -> TensorError variant (core/tensor.rs:11-53; HipError stands where CudaError stands)
_KIND = {1: "InvalidArgument", 2: "UnsupportedOperation", 3: "IdxOutOfBounds", 4: "HipError", 5: "HipError",
         6: "UnsupportedOperation", 7: "ArithmeticError", 8: "WrongDims", 9: "SizeMismatch"}


class TensorError(Exception):
    def __init__(self, status: int, msg: str):
        self.status = status
        self.kind = _KIND.get(status, "HipError")
        super().__init__(f"{self.kind}: {msg}")


def _check(status: int):
    if status != 0:
        raise TensorError(status, lib.rt_last_error().decode(errors="replace"))


def _u64s(xs: Sequence[int]):
    return (C.c_uint64 * max(len(xs), 1))(*xs)


def _i64s(xs: Sequence[int]):
    return (C.c_int64 * max(len(xs), 1))(*xs)


def _value(dtype: int, value) -> np.ndarray:
    if dtype in (U128, I128):
        return np.frombuffer((int(value) & ((1 << 128) - 1)).to_bytes(16, "little"), dtype=V16).copy()
    return np.array([value], dtype=NP_DTYPE[dtype])


class HipBuf:
    """Owns `len` elements of `dtype` in device memory; returned to the context's allocator when dropped."""

    def __init__(self, backend: "Hip", ptr: int, length: int, dtype: int):
        self.backend, self.ptr, self.len, self.dtype = backend, ptr, length, dtype

    def __del__(self):
        try:
            if self.ptr and self.backend is not None and self.backend._ctx:
                lib.rt_free(self.backend._ctx, self.ptr)
        except Exception:
            pass
        self.ptr = None

    def __eq__(self, other):                      # PartialEq of Backend::Buf
        return isinstance(other, HipBuf) and self.dtype == other.dtype and self.backend.equal(self, other)

    __hash__ = None


class Hip:
    """One context (device + stream + allocator).  `Hip.new()` mirrors `Backend::new`."""

    def __init__(self, device: int = 0):
        ctx = C.c_void_p()
        _check(lib.rt_ctx_create(device, C.byref(ctx)))
        self._ctx = ctx
        self.device = device

    @staticmethod
    def new(device: int = 0) -> "Hip":
        return Hip(device)

    def close(self):
        if self._ctx:
            lib.rt_ctx_destroy(self._ctx)
            self._ctx = None

    def sync(self):
        _check(lib.rt_sync(self._ctx))

    # ---- buffers (backend/mod.rs:225-235) --------------------------------------------------------------------------
    def alloc(self, dtype: int, length: int) -> HipBuf:
        p = C.c_void_p()
        _check(lib.rt_alloc(self._ctx, dtype, length, C.byref(p)))
        return HipBuf(self, p.value, length, dtype)

    def alloc_uninit(self, dtype: int, length: int) -> HipBuf:
        p = C.c_void_p()
        _check(lib.rt_alloc_uninit(self._ctx, dtype, length, C.byref(p)))
        return HipBuf(self, p.value, length, dtype)

    def alloc_from_slice(self, dtype: int, src: np.ndarray) -> HipBuf:
        src = np.ascontiguousarray(src, dtype=NP_DTYPE[dtype]).reshape(-1)
        p = C.c_void_p()
        _check(lib.rt_alloc_from_slice(self._ctx, dtype, src.ctypes.data_as(C.c_void_p), src.size, C.byref(p)))
        return HipBuf(self, p.value, src.size, dtype)

    def copy_from_slice(self, dst: HipBuf, src: np.ndarray):
        src = np.ascontiguousarray(src, dtype=NP_DTYPE[dst.dtype]).reshape(-1)
        _check(lib.rt_copy_from_slice(self._ctx, dst.dtype, dst.ptr, dst.len, src.ctypes.data_as(C.c_void_p), src.size))

    def copy_range_within(self, dst: HipBuf, src: HipBuf, dst_offset: int, src_offset: int, length: int):
        _check(lib.rt_copy_range_within(self._ctx, dst.dtype, dst.ptr, dst.len, src.ptr, src.len, dst_offset, src_offset, length))

    def read(self, buf: HipBuf, offset: int):
        out = np.zeros(1, dtype=NP_DTYPE[buf.dtype])
        _check(lib.rt_read(self._ctx, buf.dtype, buf.ptr, buf.len, offset, out.ctypes.data_as(C.c_void_p)))
        return out[0]

    def write(self, buf: HipBuf, offset: int, value):
        v = _value(buf.dtype, value)
        _check(lib.rt_write(self._ctx, buf.dtype, buf.ptr, buf.len, offset, v.ctypes.data_as(C.c_void_p)))

    def len(self, buf: HipBuf) -> int:
        return buf.len

    def copy(self, src: HipBuf) -> HipBuf:
        p = C.c_void_p()
        _check(lib.rt_copy(self._ctx, src.dtype, src.ptr, src.len, C.byref(p)))
        return HipBuf(self, p.value, src.len, src.dtype)

    def dump(self, src: HipBuf) -> np.ndarray:
        out = np.zeros(src.len, dtype=NP_DTYPE[src.dtype])
        _check(lib.rt_dump(self._ctx, src.dtype, src.ptr, src.len, out.ctypes.data_as(C.c_void_p)))
        return out

    def convert(self, src: HipBuf, dst: HipBuf):
        _check(lib.rt_convert(self._ctx, src.dtype, src.ptr, src.len, dst.dtype, dst.ptr, dst.len))

    def equal(self, a: HipBuf, b: HipBuf) -> bool:
        out = C.c_int32(0)
        _check(lib.rt_equal(self._ctx, a.dtype, a.ptr, a.len, b.ptr, b.len, C.byref(out)))
        return bool(out.value)

    # ---- fill / unary / scalar: the three layouts of the trait -------------------------------------------------------
    def fill_contiguous(self, buf, value, start, length):
        v = _value(buf.dtype, value)
        _check(lib.rt_fill_contiguous(self._ctx, buf.dtype, buf.ptr, buf.len, v.ctypes.data_as(C.c_void_p), start, length))

    def fill_1d_strided(self, buf, value, offset, stride, length):
        v = _value(buf.dtype, value)
        _check(lib.rt_fill_1d_strided(self._ctx, buf.dtype, buf.ptr, buf.len, v.ctypes.data_as(C.c_void_p), offset, stride, length))

    def fill_nd(self, buf, value, offset, shape, strides):
        v = _value(buf.dtype, value)
        _check(lib.rt_fill_nd(self._ctx, buf.dtype, buf.ptr, buf.len, v.ctypes.data_as(C.c_void_p), offset, len(shape), _u64s(shape), _i64s(strides)))

    def unary_contiguous(self, op: str, buf, start, length):
        _check(lib.rt_unary_contiguous(self._ctx, buf.dtype, UNARY[op], buf.ptr, buf.len, start, length))

    def unary_1d_strided(self, op: str, buf, offset, stride, length):
        _check(lib.rt_unary_1d_strided(self._ctx, buf.dtype, UNARY[op], buf.ptr, buf.len, offset, stride, length))

    def unary_nd(self, op: str, buf, offset, shape, strides):
        _check(lib.rt_unary_nd(self._ctx, buf.dtype, UNARY[op], buf.ptr, buf.len, offset, len(shape), _u64s(shape), _i64s(strides)))

    def scalar_contiguous(self, op: str, buf, value, start, length):
        v = _value(buf.dtype, value)
        _check(lib.rt_scalar_contiguous(self._ctx, buf.dtype, SCALAR[op], buf.ptr, buf.len, v.ctypes.data_as(C.c_void_p), start, length))

    def scalar_1d_strided(self, op: str, buf, value, offset, stride, length):
        v = _value(buf.dtype, value)
        _check(lib.rt_scalar_1d_strided(self._ctx, buf.dtype, SCALAR[op], buf.ptr, buf.len, v.ctypes.data_as(C.c_void_p), offset, stride, length))

    def scalar_nd(self, op: str, buf, value, offset, shape, strides):
        v = _value(buf.dtype, value)
        _check(lib.rt_scalar_nd(self._ctx, buf.dtype, SCALAR[op], buf.ptr, buf.len, v.ctypes.data_as(C.c_void_p), offset, len(shape),
                                _u64s(shape), _i64s(strides)))

    # out-of-place forms (no counterpart in the trait): dst[0 .. length) = op(src[start .. start + length))
    def unary_to(self, op: str, src, start, length, dst):
        _check(lib.rt_unary_to(self._ctx, src.dtype, UNARY[op], src.ptr, src.len, start, length, dst.ptr, dst.len))

    def scalar_to(self, op: str, src, value, start, length, dst):
        v = _value(src.dtype, value)
        _check(lib.rt_scalar_to(self._ctx, src.dtype, SCALAR[op], src.ptr, src.len, v.ctypes.data_as(C.c_void_p), start, length, dst.ptr, dst.len))

    # The trait's default methods pick one of the three layouts from |stride| contiguity (backend/mod.rs:15-213), which
    # sends a fully reversed view to the `_contiguous` loop with the offset of its *last* element.  Here the whole
    # (offset, shape, strides) goes down and the C side canonicalises it with signed strides.
    def fill(self, buf, value, meta: Tuple[int, Sequence[int], Sequence[int]]):
        self.fill_nd(buf, value, *meta)

    def apply_unary(self, op: str, buf, meta):
        self.unary_nd(op, buf, *meta)

    def scalar_apply(self, op: str, buf, value, meta):
        self.scalar_nd(op, buf, value, *meta)

    # ---- broadcast (backend/mod.rs:296-309) ----------------------------------------------------------------------------
    def broadcast(self, left: Tuple[HipBuf, tuple], right: Tuple[HipBuf, tuple], dst: Tuple[HipBuf, tuple], op: str):
        (lb, (loff, shape, lstr)), (rb, (roff, rshape, rstr)), (db, (doff, dshape, dstr)) = left, right, dst
        if list(shape) != list(rshape) or list(shape) != list(dshape):
            raise TensorError(1, f"broadcast operands must be pre-broadcast to the output shape {list(dshape)}")
        _check(lib.rt_broadcast(self._ctx, db.dtype, BINARY[op], len(shape), _u64s(shape),
                                lb.ptr, lb.len, loff, _i64s(lstr), rb.ptr, rb.len, roff, _i64s(rstr), db.ptr, db.len, doff, _i64s(dstr)))

    # ---- reductions (backend/mod.rs:357-409) -----------------------------------------------------------------------------
    def apply_reduce_contiguous_flat(self, src: HipBuf, dst: HipBuf, start: int, length: int, op: str):
        _check(lib.rt_reduce_flat(self._ctx, src.dtype, REDUCE[op], src.ptr, src.len, dst.ptr, dst.len, start, length))

    def apply_reduce_contiguous_nd(self, src: Tuple[HipBuf, tuple], dst: HipBuf, dim: int, op: str):
        sb, (off, shape, strides) = src
        _check(lib.rt_reduce_nd(self._ctx, sb.dtype, REDUCE[op], sb.ptr, sb.len, off, len(shape), _u64s(shape), _i64s(strides),
                                dst.ptr, dst.len, dim))

    def apply_reduce_contiguous_nd_static(self, src: Tuple[HipBuf, tuple], dst: HipBuf, dim: int, op: str):
        """rt_reduce_nd_static: the same reduction with its partial results in the library's built-in workspace (no allocation)."""
        sb, (off, shape, strides) = src
        _check(lib.rt_reduce_nd_static(self._ctx, sb.dtype, REDUCE[op], sb.ptr, sb.len, off, len(shape), _u64s(shape), _i64s(strides),
                                       dst.ptr, dst.len, dim))

    # Backend::apply_argmax_contiguous_flat / _nd (backend/mod.rs:412-463): dst is a u64 buffer
    def apply_argmax_contiguous_flat(self, src: HipBuf, dst: HipBuf, start: int, length: int, op: str):
        if dst.dtype != U64:
            raise TensorError(1, "argmax writes u64 indices")
        _check(lib.rt_argmax_flat(self._ctx, src.dtype, REDUCE[op], src.ptr, src.len, dst.ptr, dst.len, start, length))

    def apply_argmax_contiguous_nd(self, src: Tuple[HipBuf, tuple], dst: HipBuf, dim: int, op: str):
        if dst.dtype != U64:
            raise TensorError(1, "argmax writes u64 indices")
        sb, (off, shape, strides) = src
        _check(lib.rt_argmax_nd(self._ctx, sb.dtype, REDUCE[op], sb.ptr, sb.len, off, len(shape), _u64s(shape), _i64s(strides),
                                dst.ptr, dst.len, dim))

    def gather(self, src: HipBuf, meta, dst: HipBuf):
        off, shape, strides = meta
        _check(lib.rt_gather(self._ctx, src.dtype, src.ptr, src.len, off, len(shape), _u64s(shape), _i64s(strides), dst.ptr, dst.len))

    # ---- matmul (backend/mod.rs:474-485) ----------------------------------------------------------------------------------
    def matmul(self, lhs: Tuple[HipBuf, tuple, str], rhs: Tuple[HipBuf, tuple, str], dst: HipBuf, b: int, m: int, k: int, n: int):
        """lhs / rhs = (buffer, (offset, shape, strides), "row_major" | "column_major" | "none")."""
        (lb, (loff, lshape, lstr), lc), (rb, (roff, rshape, rstr), rc) = lhs, rhs
        _check(lib.rt_matmul(self._ctx, dst.dtype, lb.ptr, lb.len, loff, len(lshape), _u64s(lshape), _i64s(lstr), CONTIGUITY[lc],
                             rb.ptr, rb.len, roff, len(rshape), _u64s(rshape), _i64s(rstr), CONTIGUITY[rc], dst.ptr, dst.len, b, m, k, n))

    # ---- fused passes of the training step (no counterpart in the trait) --------------------------------------------------------------
    def fused_bias_relu(self, x: HipBuf, bias: HipBuf, y: HipBuf, rows: int, cols: int):
        _check(lib.rt_fused_bias_relu(self._ctx, x.dtype, x.ptr, x.len, bias.ptr, bias.len, y.ptr, y.len, rows, cols))

    def fused_l1_forward(self, y: HipBuf, target: HipBuf, gmap: HipBuf, loss: HipBuf, n: int):
        _check(lib.rt_fused_l1_forward(self._ctx, y.dtype, y.ptr, y.len, target.ptr, target.len, gmap.ptr, gmap.len, loss.ptr, loss.len, n))

    def fused_l1_relu_backward(self, gmap: HipBuf, y: HipBuf, upstream: HipBuf, dbias: HipBuf, rows: int, cols: int):
        _check(lib.rt_fused_l1_relu_backward(self._ctx, y.dtype, gmap.ptr, gmap.len, y.ptr, y.len, upstream.ptr, upstream.len, dbias.ptr, dbias.len,
                                             rows, cols))

    def fused_bias_relu_l1(self, x: HipBuf, bias: HipBuf, target: HipBuf, y: HipBuf, loss: HipBuf, rows: int, cols: int):
        _check(lib.rt_fused_bias_relu_l1(self._ctx, x.dtype, x.ptr, x.len, bias.ptr, bias.len, target.ptr, target.len, y.ptr, y.len, loss.ptr, loss.len,
                                         rows, cols))

    def fused_l1_relu_backward_t(self, y: HipBuf, target: HipBuf, upstream: HipBuf, dbias: HipBuf, rows: int, cols: int):
        _check(lib.rt_fused_l1_relu_backward_t(self._ctx, y.dtype, y.ptr, y.len, target.ptr, target.len, upstream.ptr, upstream.len, dbias.ptr, dbias.len,
                                               rows, cols))

    def fused_chain(self, inputs, steps, dst: HipBuf, length: int, dst_start: int = 0):
        """rt_fused_chain: `inputs` = [(buffer, start), ...]; `steps` = [("unary", op), ("scalar", op, value), ("binary", op, k),
        ("binary_rev", op, k)] with k an index into `inputs`; dst[dst_start + i] = steps(inputs[0][start0 + i]) for i < length."""
        dtype = dst.dtype
        n = len(inputs)
        ptrs = (C.c_void_p * max(n, 1))(*[b.ptr for b, _ in inputs])
        lens = _u64s([b.len for b, _ in inputs])
        starts = _u64s([st for _, st in inputs])
        arr = (_ffi.ChainStep * max(len(steps), 1))()
        for i, st in enumerate(steps):
            kind = {"unary": 0, "scalar": 1, "binary": 2, "binary_rev": 3}[st[0]]
            arr[i].kind = kind
            arr[i].op = (UNARY, SCALAR, BINARY, BINARY)[kind][st[1]]
            if kind == 1:
                raw = _value(dtype, st[2]).tobytes()
                for j, byte in enumerate(raw[:8]):
                    arr[i].value[j] = byte
            elif kind >= 2:
                arr[i].operand = st[2]
        _check(lib.rt_fused_chain(self._ctx, dtype, n, ptrs, lens, starts, length, len(steps), arr, dst.ptr, dst.len, dst_start))

    # ---- timing -----------------------------------------------------------------------------------------------------------
    def event(self):
        e = C.c_void_p()
        _check(lib.rt_event_create(self._ctx, C.byref(e)))
        return e

    def record(self, ev):
        _check(lib.rt_event_record(self._ctx, ev))

    def elapsed_ms(self, start, stop) -> float:
        out = C.c_float(0)
        _check(lib.rt_event_elapsed_ms(self._ctx, start, stop, C.byref(out)))
        return out.value

    def mem_stats(self):
        a, b, c = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
        _check(lib.rt_mem_stats(self._ctx, C.byref(a), C.byref(b), C.byref(c)))
        return {"in_use": a.value, "cached": b.value, "device_allocs": c.value}

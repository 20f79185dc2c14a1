"""Python face of the C++ host layer (rtensors_amd/host/*.hpp through librt_host.so): tensors, views, operators,
reductions and the autograd training step on the Hip backend.  Method names follow the reference's tensor API
(from_buf, slice, permute, transpose, unsqueeze_at, squeeze, owned, contiguous, sum_at, ...)."""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

from .hip import BINARY, DTYPE_BY_NAME, NP_DTYPE, REDUCE, SCALAR, UNARY

_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "librt_host.so")
if not os.path.exists(_LIB):
    raise ImportError(f"{_LIB} is missing: build it with `python -m rtensors_amd.build`")
_h = C.CDLL(_LIB)
_h.rth_last_error.restype = C.c_char_p
for _n in ("rth_backend_destroy", "rth_free"):
    getattr(_h, _n).restype = None
    getattr(_h, _n).argtypes = [C.c_void_p]

_KINDS = ["InvalidShape", "InvalidDim", "IdxOutOfBounds", "WrongDims", "BroadcastError", "SizeMismatch", "UnsupportedOperation",
          "GradError", "HipError", "Panic", "ContiguityError"]
MAX_RANK = 128


class TensorError(Exception):
    def __init__(self, code: int, msg: str):
        self.kind = _KINDS[code - 1] if 1 <= code <= len(_KINDS) else "HipError"
        super().__init__(msg)


def _ck(code: int):
    if code != 0:
        raise TensorError(code, _h.rth_last_error().decode(errors="replace"))


def _u64(xs):
    return (C.c_uint64 * max(len(xs), 1))(*[int(x) for x in xs])


def _i64(xs):
    return (C.c_int64 * max(len(xs), 1))(*[int(x) for x in xs])


class Slice:
    """core/slice.rs:17-115."""

    def __init__(self, start: Optional[int] = None, end: Optional[int] = None, step: int = 1):
        self.start, self.end, self.step = start, end, step

    @staticmethod
    def full(): return Slice(None, None, 1)
    @staticmethod
    def index(i): return Slice(i, i, 1)
    @staticmethod
    def range(a, b): return Slice(a, b, -1 if a > b else 1)

    @staticmethod
    def range_inclusive(a, b):
        step = -1 if a > b else 1
        if step < 0:
            return Slice(a, b - 1 if b > 0 else None, step)
        return Slice(a, b + 1, step)

    def _args(self):
        return (1 if self.start is not None else 0, self.start or 0, 1 if self.end is not None else 0, self.end or 0, self.step)


# ---- metadata-only entry points (no device needed) ---------------------------------------------------------------------
def _meta_out():
    return C.c_int(0), (C.c_uint64 * MAX_RANK)(), (C.c_int64 * MAX_RANK)(), C.c_uint64(0)


def _meta_ret(r, sh, st, off):
    n = r.value
    return list(sh[:n]), list(st[:n]), off.value


def meta_slice(shape, strides, offset, dim, sl: Slice):
    r, sh, st, off = _meta_out()
    _ck(_h.rth_meta_slice(len(shape), _u64(shape), _i64(strides), C.c_uint64(offset), C.c_uint64(dim), *[C.c_int(sl._args()[0]), C.c_uint64(sl._args()[1]),
        C.c_int(sl._args()[2]), C.c_uint64(sl._args()[3]), C.c_int64(sl._args()[4])], C.byref(r), sh, st, C.byref(off)))
    return _meta_ret(r, sh, st, off)


def meta_permute(shape, strides, offset, dims):
    r, sh, st, off = _meta_out()
    _ck(_h.rth_meta_permute(len(shape), _u64(shape), _i64(strides), C.c_uint64(offset), len(dims), _u64(dims), C.byref(r), sh, st, C.byref(off)))
    return _meta_ret(r, sh, st, off)


def meta_unsqueeze(shape, strides, offset, dim):
    r, sh, st, off = _meta_out()
    _ck(_h.rth_meta_unsqueeze(len(shape), _u64(shape), _i64(strides), C.c_uint64(offset), C.c_uint64(dim), C.byref(r), sh, st, C.byref(off)))
    return _meta_ret(r, sh, st, off)


def meta_squeeze(shape, strides, offset, dim: Optional[int]):
    r, sh, st, off = _meta_out()
    _ck(_h.rth_meta_squeeze(len(shape), _u64(shape), _i64(strides), C.c_uint64(offset), C.c_int64(-1 if dim is None else dim), C.byref(r), sh, st, C.byref(off)))
    return _meta_ret(r, sh, st, off)


def meta_broadcast(shape_a, strides_a, shape_b, strides_b):
    r = C.c_int(0)
    sh, sa, sb = (C.c_uint64 * MAX_RANK)(), (C.c_int64 * MAX_RANK)(), (C.c_int64 * MAX_RANK)()
    _ck(_h.rth_meta_broadcast(len(shape_a), _u64(shape_a), _i64(strides_a), len(shape_b), _u64(shape_b), _i64(strides_b), C.byref(r), sh, sa, sb))
    n = r.value
    return list(sh[:n]), list(sa[:n]), list(sb[:n])


def meta_contiguity_type(shape, strides) -> str:
    return ("row_major", "column_major", "none")[_h.rth_meta_contiguity_type(len(shape), _u64(shape), _i64(strides))]


def meta_is_contiguous(shape, strides) -> bool:
    return bool(_h.rth_meta_is_contiguous(len(shape), _u64(shape), _i64(strides)))


# ---- device tensors ---------------------------------------------------------------------------------------------------------
class Backend:
    def __init__(self, device: int = 0):
        p = C.c_void_p()
        _ck(_h.rth_backend_create(device, C.byref(p)))
        self._p = p

    def sync(self):
        _ck(_h.rth_backend_sync(self._p))


class Tensor:
    def __init__(self, handle, backend: Backend):
        self._p, self.backend = handle, backend
        self.last_path = None

    def __del__(self):
        try:
            if self._p:
                _h.rth_free(self._p)
        except Exception:
            pass
        self._p = None

    @staticmethod
    def from_buf(backend: Backend, dtype, values, shape: Sequence[int]) -> "Tensor":
        code = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else dtype
        arr = np.ascontiguousarray(np.asarray(values).astype(NP_DTYPE[code]).reshape(-1))
        p = C.c_void_p()
        _ck(_h.rth_from_buf(backend._p, code, arr.ctypes.data_as(C.c_void_p), C.c_uint64(arr.size), len(shape), _u64(shape), C.byref(p)))
        return Tensor(p, backend)

    @staticmethod
    def zeros(backend, dtype, shape):
        code = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else dtype
        p = C.c_void_p(); _ck(_h.rth_zeros(backend._p, code, len(shape), _u64(shape), C.byref(p))); return Tensor(p, backend)

    @staticmethod
    def ones(backend, dtype, shape):
        code = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else dtype
        p = C.c_void_p(); _ck(_h.rth_ones(backend._p, code, len(shape), _u64(shape), C.byref(p))); return Tensor(p, backend)

    @staticmethod
    def max_of(backend, dtype, shape):
        """`TensorBase::max(shape)` (core/primitives.rs:490-495): every element T::MAX."""
        code = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else dtype
        p = C.c_void_p(); _ck(_h.rth_limit(backend._p, code, 1, len(shape), _u64(shape), C.byref(p))); return Tensor(p, backend)

    @staticmethod
    def min_of(backend, dtype, shape):
        """`TensorBase::min(shape)` (core/primitives.rs:501-506): every element T::MIN."""
        code = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else dtype
        p = C.c_void_p(); _ck(_h.rth_limit(backend._p, code, 0, len(shape), _u64(shape), C.byref(p))); return Tensor(p, backend)

    @staticmethod
    def scalar(backend, dtype, value): return Tensor.from_buf(backend, dtype, [value], [])            # core/primitives.rs:418-420

    @staticmethod
    def column(backend, dtype, values): return Tensor.from_buf(backend, dtype, values, [len(values)])  # core/primitives.rs:428-432

    @staticmethod
    def row(backend, dtype, values): return Tensor.from_buf(backend, dtype, values, [1, len(values)])  # core/primitives.rs:440-444

    def into_dtype(self, dtype):
        """`TensorBase::into_dtype::<N>()` (core/primitives.rs:527-539): the whole buffer converted, same meta."""
        code = DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else dtype
        return self._new(_h.rth_into_dtype, C.c_int(code))

    def _info(self):
        r, sh, st, off = _meta_out()
        dt, iv, cg, bl = C.c_int(0), C.c_int(0), C.c_int(0), C.c_uint64(0)
        _ck(_h.rth_info(self._p, C.byref(r), sh, st, C.byref(off), C.byref(dt), C.byref(iv), C.byref(cg), C.byref(bl)))
        n = r.value
        return {"shape": list(sh[:n]), "strides": list(st[:n]), "offset": off.value, "dtype": dt.value, "is_view": bool(iv.value),
                "contiguous": bool(cg.value), "buf_len": bl.value}

    shape = property(lambda self: self._info()["shape"])
    strides = property(lambda self: self._info()["strides"])
    offset = property(lambda self: self._info()["offset"])
    dtype = property(lambda self: self._info()["dtype"])

    def is_contiguous(self): return self._info()["contiguous"]

    def _new(self, fn, *args):
        p = C.c_void_p()
        _ck(fn(self._p, *args, C.byref(p)))
        return Tensor(p, self.backend)

    def slice(self, dim, sl):
        if isinstance(sl, int):
            sl = Slice.index(sl)
        a = sl._args()
        return self._new(_h.rth_slice, C.c_uint64(dim), C.c_int(a[0]), C.c_uint64(a[1]), C.c_int(a[2]), C.c_uint64(a[3]), C.c_int64(a[4]))

    def permute(self, dims): return self._new(_h.rth_permute, len(dims), _u64(dims))
    def transpose(self): return self._new(_h.rth_transpose)
    def unsqueeze_at(self, d): return self._new(_h.rth_unsqueeze, C.c_uint64(d))
    def squeeze_at(self, d): return self._new(_h.rth_squeeze, C.c_int64(d))
    def squeeze(self): return self._new(_h.rth_squeeze, C.c_int64(-1))
    def view_as(self, shape): return self._new(_h.rth_view_as, len(shape), _u64(shape))       # core/tensor.rs:120-122
    def reshape(self, shape): return self._new(_h.rth_reshape, len(shape), _u64(shape))       # core/tensor.rs:238-243
    def owned(self): return self._new(_h.rth_owned)
    def contiguous(self): return self._new(_h.rth_contiguous)

    def _bin(self, o, op, assign):
        if isinstance(o, Tensor):
            if assign:
                _ck(_h.rth_binary_assign(self._p, o._p, BINARY[op])); return self
            return self._new(_h.rth_binary, o._p, BINARY[op])
        if assign:
            _ck(_h.rth_scalar_assign(self._p, SCALAR[op], C.c_double(o))); return self
        return self._new(_h.rth_scalar, SCALAR[op], C.c_double(o))

    def __add__(self, o): return self._bin(o, "add", False)
    def __sub__(self, o): return self._bin(o, "sub", False)
    def __mul__(self, o): return self._bin(o, "mul", False)
    def __truediv__(self, o): return self._bin(o, "div", False)
    def __iadd__(self, o): return self._bin(o, "add", True)
    def __isub__(self, o): return self._bin(o, "sub", True)
    def __imul__(self, o): return self._bin(o, "mul", True)
    def __itruediv__(self, o): return self._bin(o, "div", True)
    def __neg__(self): return self.unary("neg")

    def unary(self, op): return self._new(_h.rth_unary, UNARY[op])
    def unary_inplace(self, op): _ck(_h.rth_unary_inplace(self._p, UNARY[op])); return self
    def scalar_op_inplace(self, op, v): _ck(_h.rth_scalar_assign(self._p, SCALAR[op], C.c_double(v))); return self
    def relu(self): return self.unary("relu")
    def sign(self): return self.unary("sign")
    def abs(self): return self.unary("abs")

    def matmul(self, o): return self._new(_h.rth_matmul, o._p)
    def dot(self, o): return self._new(_h.rth_dot, o._p)
    def outer(self, o): return self._new(_h.rth_outer, o._p)

    def reduce(self, op, axis=None): return self._new(_h.rth_reduce, REDUCE[op], C.c_int64(-1 if axis is None else axis))
    def sum_at(self, a): return self.reduce("sum", a)
    def mean_at(self, a): return self.reduce("mean", a)
    def max_at(self, a): return self.reduce("max", a)
    def min_at(self, a): return self.reduce("min", a)
    def sum(self): return self.reduce("sum")
    def mean(self): return self.reduce("mean")
    def max(self): return self.reduce("max")
    def min(self): return self.reduce("min")
    # the kinds only the reference's Cuda backend implements (ops/reduction/mod.rs:411-500); argmax / argmin give u64 tensors
    def var_at(self, a): return self.reduce("var", a)
    def pop_var_at(self, a): return self.reduce("pop_var", a)
    def std_at(self, a, unbiased): return self.reduce("std" if unbiased else "pop_std", a)
    def norm_at(self, a, norm): return self.reduce({"L1": "l1_norm", "L2": "l2_norm"}[norm], a)
    def l1_norm_at(self, a): return self.reduce("l1_norm", a)
    def l2_norm_at(self, a): return self.reduce("l2_norm", a)
    def logsumexp_at(self, a): return self.reduce("logsumexp", a)
    def argmax_at(self, a): return self.reduce("argmax", a)
    def argmin_at(self, a): return self.reduce("argmin", a)
    def var(self): return self.reduce("var")
    def pop_var(self): return self.reduce("pop_var")
    def std(self, unbiased): return self.reduce("std" if unbiased else "pop_std")
    def norm(self, norm): return self.reduce({"L1": "l1_norm", "L2": "l2_norm"}[norm])
    def logsumexp(self): return self.reduce("logsumexp")
    def argmax(self): return self.reduce("argmax")
    def argmin(self): return self.reduce("argmin")

    def fill(self, v): _ck(_h.rth_fill(self._p, C.c_double(v)))

    def get(self, idx):
        out = C.c_double(0)
        _ck(_h.rth_get(self._p, len(idx), _u64(idx), C.byref(out)))
        return out.value

    def set(self, idx, v): _ck(_h.rth_set(self._p, len(idx), _u64(idx), C.c_double(v)))

    def to_numpy(self) -> np.ndarray:
        info = self._info()
        n = int(np.prod(info["shape"], dtype=np.int64)) if info["shape"] else 1
        out = np.zeros(n, dtype=NP_DTYPE[info["dtype"]])
        _ck(_h.rth_to_host(self._p, out.ctypes.data_as(C.c_void_p)))
        return out.reshape(info["shape"])

    def dump_buffer(self) -> np.ndarray:
        info = self._info()
        out = np.zeros(info["buf_len"], dtype=NP_DTYPE[info["dtype"]])
        _ck(_h.rth_dump_buffer(self._p, out.ctypes.data_as(C.c_void_p)))
        return out

    def equals(self, o) -> bool:
        r = C.c_int(0)
        _ck(_h.rth_equals(self._p, o._p, C.byref(r)))
        return bool(r.value)


class Expr:
    """A pending elementwise expression (rt::Expr of the host layer): the operators are recorded, `eval()` issues them as fused
    passes where the operands allow (every operand read once, the result written once) and as the ordinary operators elsewhere.
    `lazy(a) * 3.0 + b` ... `.relu()` ... `- 1.0` ... `.eval()`; `fused_launches` holds the number of fused launches of the last eval."""

    def __init__(self, first: Tensor, steps=()):
        self.first, self.steps, self.fused_launches = first, list(steps), None

    def _with(self, step): return Expr(self.first, self.steps + [step])

    def _bin(self, o, op, rev=False):
        if isinstance(o, Tensor):
            return self._with((3 if rev else 2, BINARY[op], 0.0, o))
        if rev:
            raise TypeError("scalar op expression is not an operator of the reference")
        return self._with((1, SCALAR[op], float(o), None))

    def __add__(self, o): return self._bin(o, "add")
    def __sub__(self, o): return self._bin(o, "sub")
    def __mul__(self, o): return self._bin(o, "mul")
    def __truediv__(self, o): return self._bin(o, "div")
    def rsub(self, t: Tensor): return self._bin(t, "sub", True)
    def rdiv(self, t: Tensor): return self._bin(t, "div", True)
    def unary(self, op): return self._with((0, UNARY[op], 0.0, None))
    def scalar(self, op, v): return self._with((1, SCALAR[op], float(v), None))
    def relu(self): return self.unary("relu")
    def abs(self): return self.unary("abs")
    def __neg__(self): return self.unary("neg")

    def eval(self) -> Tensor:
        n = len(self.steps)
        kinds = (C.c_int * max(n, 1))(*[s[0] for s in self.steps])
        ops = (C.c_int * max(n, 1))(*[s[1] for s in self.steps])
        vals = (C.c_double * max(n, 1))(*[s[2] for s in self.steps])
        opnds = (C.c_void_p * max(n, 1))(*[s[3]._p if s[3] is not None else None for s in self.steps])
        p, fused = C.c_void_p(), C.c_int(0)
        _ck(_h.rth_expr_eval(self.first._p, n, kinds, ops, vals, opnds, C.byref(p), C.byref(fused)))
        self.fused_launches = fused.value
        return Tensor(p, self.first.backend)


def lazy(t: Tensor) -> Expr:
    return Expr(t)


def train_step(x: Tensor, bias: Tensor, target: Tensor, lr: float, mode: str = "sum", seed_with_loss: bool = True):
    """y = relu(x + bias); loss = mean_l1_loss(y, target); backward; SGD(lr) on bias in place.  Returns (loss, d_bias).
    mode 'sum' sums the upstream gradient over the broadcast dim; 'reference_literal' reproduces grad/backwards.rs:527."""
    pl, pg = C.c_void_p(), C.c_void_p()
    _ck(_h.rth_train_step(x._p, bias._p, target._p, C.c_double(lr), 0 if mode == "sum" else 1, 1 if seed_with_loss else 0, C.byref(pl), C.byref(pg)))
    return Tensor(pl, x.backend), Tensor(pg, x.backend)


def train_step_fused(x: Tensor, bias: Tensor, target: Tensor, lr: float, seed_with_loss: bool = True, passes: int = 2):
    """The same step through the fused passes (rt_fused_*): passes=2 forms the L1 gradient map in registers, passes=3 stores it as
    the tape does.  Returns (loss, d_bias, used_fused); operands the fused form does
    not take (views, dtypes other than f32 / f64, rows that are not whole 16-byte vectors) go through the tape and used_fused is False."""
    pl, pg, used = C.c_void_p(), C.c_void_p(), C.c_int(0)
    _ck(_h.rth_train_step_fused(x._p, bias._p, target._p, C.c_double(lr), 1 if seed_with_loss else 0, int(passes), C.byref(pl), C.byref(pg), C.byref(used)))
    return Tensor(pl, x.backend), Tensor(pg, x.backend), bool(used.value)


def linear_step(x: Tensor, w: Tensor, target: Tensor, lr: float, seed_with_loss: bool = True):
    """y = x @ w; loss = mean_l1_loss(y, target); backward; SGD(lr) on w in place.  Returns (loss, d_w)."""
    pl, pg = C.c_void_p(), C.c_void_p()
    _ck(_h.rth_linear_step(x._p, w._p, target._p, C.c_double(lr), 1 if seed_with_loss else 0, C.byref(pl), C.byref(pg)))
    return Tensor(pl, x.backend), Tensor(pg, x.backend)

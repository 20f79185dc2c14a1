"""TEST INFRASTRUCTURE ONLY -- never imported by the product path.

Restatement of the operator glue that sits between user code and the `Backend` trait in the reference:
which backend call each operator issues and with which (offset, shape, strides).  Data loops are the C++
oracle (oracle/cpu.py); this file only sequences them.  Paths are relative to libs/rtensors/src/.

An `OTensor` stands for `TensorBase` (owns its buffer) or, when `is_view` is set, for
`TensorView`/`TensorViewMut` (shares the buffer of the tensor it was taken from).
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np

from . import cpu
from .meta import (MetaTensor, Slice, TensorError, compute_broadcasted_params, compute_permuted_parameters, contiguity_type,
                   compute_sliced_parameters, compute_squeezed_parameters, compute_unsqueezed_parameters, compute_view_as_parameters,
                   logical_to_buffer_idx, reduction_output_meta, shape_to_stride)


class OTensor:
    def __init__(self, dtype: int, buf: np.ndarray, meta: MetaTensor, is_view: bool = False):
        self.dtype = dtype
        self.buf = buf
        self.meta = meta
        self.is_view = is_view
        self.last_path = None      # which of the three layout loops the last in-place op dispatched to

    # ---- constructors: core/primitives.rs:367-506 -----------------------------------------------------------
    @staticmethod
    def from_buf(dtype, values, shape: Sequence[int]) -> "OTensor":
        """`TensorBase::from_buf(vec, shape)`: row-major, offset 0; length must match the shape."""
        if isinstance(dtype, str):
            dtype = cpu.DTYPE_BY_NAME[dtype]
        buf = values.astype(cpu.NP_DTYPE[dtype]).reshape(-1).copy() if isinstance(values, np.ndarray) \
            else cpu.from_ints(dtype, values)
        meta = MetaTensor.row_major(list(shape))
        if buf.size != meta.size():
            raise TensorError("InvalidShape", f"{buf.size} elements for shape {list(shape)}")
        return OTensor(dtype, buf, meta)

    @staticmethod
    def zeros(dtype, shape) -> "OTensor":
        if isinstance(dtype, str):
            dtype = cpu.DTYPE_BY_NAME[dtype]
        meta = MetaTensor.row_major(list(shape))
        return OTensor(dtype, np.zeros(meta.size(), dtype=cpu.NP_DTYPE[dtype]), meta)

    # ---- metadata-only views: core/tensor.rs:548-628 ------------------------------------------------------------
    def _view(self, shape, strides, offset) -> "OTensor":
        return OTensor(self.dtype, self.buf, MetaTensor(list(shape), list(strides), offset), is_view=True)

    def view(self) -> "OTensor":
        return self._view(self.meta.shape, self.meta.strides, self.meta.offset)

    def slice(self, dim: int, sl) -> "OTensor":
        if isinstance(sl, int):
            sl = Slice.index(sl)
        shape, strides, offset = compute_sliced_parameters(self.meta.shape, self.meta.strides, self.meta.offset, dim, sl)
        return self._view(shape, strides, offset)

    def permute(self, dims) -> "OTensor":
        shape, strides = compute_permuted_parameters(self.meta.shape, self.meta.strides, list(dims))
        return self._view(shape, strides, self.meta.offset)

    def transpose(self) -> "OTensor":
        return self.permute(list(range(self.meta.rank() - 1, -1, -1)))

    def unsqueeze_at(self, dim: int) -> "OTensor":
        shape, strides = compute_unsqueezed_parameters(self.meta.shape, self.meta.strides, dim)
        return self._view(shape, strides, self.meta.offset)

    def squeeze_at(self, dim: int) -> "OTensor":
        shape, strides = compute_squeezed_parameters(self.meta.shape, self.meta.strides, dim)
        return self._view(shape, strides, self.meta.offset)

    def squeeze(self) -> "OTensor":
        shape, strides = compute_squeezed_parameters(self.meta.shape, self.meta.strides, None)
        return self._view(shape, strides, self.meta.offset)

    def view_as(self, shape) -> "OTensor":
        """core/tensor.rs:120-122, 328-355: reinterpret a contiguous layout under another shape (no copy)."""
        return self._view(*compute_view_as_parameters(self.meta, list(shape)))

    def reshape(self, shape) -> "OTensor":
        """core/tensor.rs:238-243: `contiguous()` then the `view_as` meta on the new owner."""
        c = self.contiguous()
        sh, st, off = compute_view_as_parameters(c.meta, list(shape))
        return OTensor(c.dtype, c.buf, MetaTensor(sh, st, off))

    # ---- element access: core/tensor.rs:535-541, 665-682; backend/cpu.rs:185-207 -----------------------------------
    def get(self, idx):
        b = logical_to_buffer_idx(list(idx), self.meta.strides, self.meta.offset)
        if b >= self.buf.size:
            raise TensorError("IdxOutOfBounds", f"index {b} out of bounds for buffer of length {self.buf.size}")
        return self.buf[b]

    def set(self, idx, value):
        b = logical_to_buffer_idx(list(idx), self.meta.strides, self.meta.offset)
        if b >= self.buf.size:
            raise TensorError("IdxOutOfBounds", f"index {b} out of bounds for buffer of length {self.buf.size}")
        self.buf[b] = value

    def fill(self, value):
        cpu.fill(self.dtype, self.buf, value, self.meta)

    # ---- owned / contiguous: core/tensor.rs:215-325; core/primitives.rs:68-81 ------------------------------------
    def owned(self) -> "OTensor":
        """TensorBase: clone of the whole buffer with the same meta.  Views: gather into a fresh row-major buffer."""
        if not self.is_view:
            return OTensor(self.dtype, self.buf.copy(), MetaTensor(list(self.meta.shape), list(self.meta.strides), self.meta.offset))
        return self._gathered()

    def contiguous(self) -> "OTensor":
        if not self.is_view and self.meta.is_contiguous():
            return self.owned()
        return self._gathered()

    def _gathered(self) -> "OTensor":
        out = cpu.gather(self.dtype, self.buf, self.meta)
        return OTensor(self.dtype, out, MetaTensor.row_major(self.meta.shape))

    def to_numpy(self) -> np.ndarray:
        """Row-major values of the elements this tensor/view addresses, shaped like the tensor."""
        return cpu.gather(self.dtype, self.buf, self.meta).reshape(self.meta.shape)

    # ---- matmul / dot / outer: ops/linalg/matmul.rs:5-180 ------------------------------------------------------------------
    def matmul(self, other: "OTensor") -> "OTensor":
        lhs, rhs = self, other
        if lhs.meta.rank() < 2:
            raise TensorError("InvalidShape", "LHS tensor must have rank >= 2 for matmul")
        if rhs.meta.rank() < 2:
            raise TensorError("InvalidShape", "RHS tensor must have rank >= 2 for matmul")
        # an operand whose last two dims have no unit stride (or whose batch dims do not collapse) is made row-major first;
        # negative strides are treated the same way here (the reference casts them to usize)
        def prepared(t):
            ct = contiguity_type(t.meta)
            if ct == "none" or any(s < 0 for s in t.meta.strides):
                return t.contiguous()
            return t
        lhs, rhs = prepared(lhs), prepared(rhs)
        lr, rr = lhs.meta.rank(), rhs.meta.rank()
        if lr != rr:
            raise TensorError("InvalidShape", f"Both tensors must have the same rank >= 2, got lhs rank {lr} and rhs rank {rr}")
        lb, rb = list(lhs.meta.shape[:lr - 2]), list(rhs.meta.shape[:rr - 2])
        if lb != rb:
            raise TensorError("SizeMismatch", f"Batch dimensions must match for matmul, got {lb} and {rb}")
        b = 1
        for d in lb:
            b *= d
        m, k_l = lhs.meta.shape[lr - 2], lhs.meta.shape[lr - 1]
        k_r, n = rhs.meta.shape[rr - 2], rhs.meta.shape[rr - 1]
        if k_l != k_r:
            raise TensorError("SizeMismatch", f"Inner matrix dimensions must match for matmul, got lhs K={k_l} and rhs K={k_r}")
        # the kernels step through batches by strides[rank - 3] alone: collapse flat batch dims to that stride
        out = cpu.matmul(self.dtype, lhs.buf, lhs.meta, rhs.buf, rhs.meta, b, m, k_l, n)
        return OTensor(self.dtype, out, MetaTensor.row_major(lb + [m, n]))

    def dot(self, other: "OTensor") -> "OTensor":
        if self.meta.rank() != 1 or other.meta.rank() != 1:
            raise TensorError("InvalidShape", "Dot product is only defined for 1-D tensors")
        return self.unsqueeze_at(0).matmul(other.unsqueeze_at(1)).squeeze()

    def outer(self, other: "OTensor") -> "OTensor":
        if self.meta.rank() != 1 or other.meta.rank() != 1:
            raise TensorError("InvalidShape", "Outer product is only defined for 1-D tensors")
        return self.unsqueeze_at(1).matmul(other.unsqueeze_at(0))

    # ---- broadcast binary operators: ops/broadcast/add.rs:7-478 (sub/mul/div are textual twins) ---------------------
    def _binary(self, other: "OTensor", op: str) -> "OTensor":
        out_shape, stra, strb = compute_broadcasted_params(self.meta, other.meta)
        result = OTensor.zeros(self.dtype, out_shape)                     # zeros_on(backend, out_shape)
        meta_a = MetaTensor(out_shape, stra, self.meta.offset)
        meta_b = MetaTensor(out_shape, strb, other.meta.offset)
        cpu.broadcast(self.dtype, op, self.buf, meta_a, other.buf, meta_b, result.buf, result.meta)
        return result

    def _binary_assign(self, other: "OTensor", op: str) -> "OTensor":
        out_shape, stra, strb = compute_broadcasted_params(self.meta, other.meta)
        if list(self.meta.shape) != list(out_shape):
            raise TensorError("Panic", f"incompatible shapes for in-place op: {other.meta.shape} does not broadcast to {self.meta.shape}")
        meta_a = MetaTensor(out_shape, stra, self.meta.offset)
        meta_b = MetaTensor(out_shape, strb, other.meta.offset)
        cpu.broadcast(self.dtype, op, self.buf, meta_a, other.buf, meta_b, self.buf, meta_a)
        return self

    # ---- scalar operators: ops/scalar/add.rs:20-121 (sub/mul/div are twins) ------------------------------------
    def _scalar_assign(self, value, op: str) -> "OTensor":
        self.last_path = cpu.scalar(self.dtype, op, self.buf, value, self.meta)
        return self

    def _scalar(self, value, op: str) -> "OTensor":
        result = self.owned()
        return result._scalar_assign(value, op)

    def _dispatch_bin(self, other, op, assign):
        if isinstance(other, OTensor):
            return self._binary_assign(other, op) if assign else self._binary(other, op)
        return self._scalar_assign(other, op) if assign else self._scalar(other, op)

    def __add__(self, o): return self._dispatch_bin(o, "add", False)
    def __sub__(self, o): return self._dispatch_bin(o, "sub", False)
    def __mul__(self, o): return self._dispatch_bin(o, "mul", False)
    def __truediv__(self, o): return self._dispatch_bin(o, "div", False)
    def __iadd__(self, o): return self._dispatch_bin(o, "add", True)
    def __isub__(self, o): return self._dispatch_bin(o, "sub", True)
    def __imul__(self, o): return self._dispatch_bin(o, "mul", True)
    def __itruediv__(self, o): return self._dispatch_bin(o, "div", True)

    def __neg__(self):                                                   # ops/unary/mod.rs:314-396
        return self.unary("neg")

    # ---- unary ops: ops/unary/mod.rs:56-126 -----------------------------------------------------------------------
    def unary_inplace(self, op: str) -> "OTensor":
        self.last_path = cpu.unary(self.dtype, op, self.buf, self.meta)
        return self

    def unary(self, op: str) -> "OTensor":
        result = self.owned()
        return result.unary_inplace(op)

    def scalar_op_inplace(self, op: str, value) -> "OTensor":            # leaky_relu / elu / log / log1p, ops/scalar/mod.rs:142-170
        cpu.scalar(self.dtype, op, self.buf, value, self.meta)
        return self

    # ---- reductions: ops/reduction/mod.rs:262-302, 346-408 ------------------------------------------------------------
    def reduce(self, op: str, axis: Optional[int] = None, honour_offset: bool = True) -> "OTensor":
        t = self if self.meta.is_contiguous() else self.contiguous()
        if op in cpu.STAT_OPS or op in cpu.ARG_OPS:                        # do_reduce / do_argmax with the Cuda backend's kinds
            arg = op in cpu.ARG_OPS
            if axis is not None and not (0 <= axis < t.meta.rank()):
                raise TensorError("InvalidDim", "reduction axis out of range")
            out = (cpu.argmax if arg else cpu.reduce_stat)(t.dtype, op, t.buf, t.meta, axis)
            out_meta = MetaTensor([], [], 0) if axis is None else reduction_output_meta(t.meta, axis)
            return OTensor(cpu.U64 if arg else t.dtype, out, out_meta)
        if axis is None:                                                  # Idx::Item
            out = cpu.reduce_flat(t.dtype, op, t.buf, t.meta.offset, t.meta.size())
            return OTensor(t.dtype, out, MetaTensor([], [], 0))
        out_meta = reduction_output_meta(t.meta, axis)
        if t.meta.rank() == 1:                                            # backend/mod.rs:392-399
            out = cpu.reduce_flat(t.dtype, op, t.buf, t.meta.offset, t.meta.size())
        else:
            out = cpu.reduce_nd(t.dtype, op, t.buf, t.meta, axis, honour_offset=honour_offset)
        return OTensor(t.dtype, out, out_meta)

    def sum_at(self, axis): return self.reduce("sum", axis)
    def mean_at(self, axis): return self.reduce("mean", axis)
    def max_at(self, axis): return self.reduce("max", axis)
    def min_at(self, axis): return self.reduce("min", axis)
    def prod_at(self, axis): return self.reduce("prod", axis)
    def sum(self): return self.reduce("sum")
    def mean(self): return self.reduce("mean")
    def max(self): return self.reduce("max")
    def min(self): return self.reduce("min")
    def prod(self): return self.reduce("prod")
    def var_at(self, axis): return self.reduce("var", axis)
    def pop_var_at(self, axis): return self.reduce("pop_var", axis)
    def std_at(self, axis, unbiased): return self.reduce("std" if unbiased else "pop_std", axis)
    def norm_at(self, axis, norm): return self.reduce({"L1": "l1_norm", "L2": "l2_norm"}[norm], axis)
    def logsumexp_at(self, axis): return self.reduce("logsumexp", axis)
    def argmax_at(self, axis): return self.reduce("argmax", axis)
    def argmin_at(self, axis): return self.reduce("argmin", axis)
    def var(self): return self.reduce("var")
    def pop_var(self): return self.reduce("pop_var")
    def std(self, unbiased): return self.reduce("std" if unbiased else "pop_std")
    def norm(self, norm): return self.reduce({"L1": "l1_norm", "L2": "l2_norm"}[norm])
    def logsumexp(self): return self.reduce("logsumexp")
    def argmax(self): return self.reduce("argmax")
    def argmin(self): return self.reduce("argmin")


def mean_l1_loss(y: OTensor, target: OTensor):
    """ops/broadcast/l1.rs:49-84: returns (loss, grad_map) with grad_map = sign(sign(y - t)) / N."""
    diff = y - target
    gmap = diff.unary("sign")
    diff.unary_inplace("abs")
    loss = diff.mean()
    n = np.float32(diff.meta.size())                                      # T::from_usize goes through f32
    grad_map = gmap.unary("sign") / cpu.NP_DTYPE[y.dtype].type(n)
    return loss, grad_map


def relu_grad_map(inp: OTensor) -> OTensor:
    """ops/unary/mod.rs:234-252: zeros, then 1 where `input > 0` (the reference does it with one get/set per element)."""
    vals = inp.to_numpy().reshape(-1)
    out = np.where(vals > 0, 1, 0).astype(vals.dtype)
    return OTensor(inp.dtype, out, MetaTensor.row_major(inp.meta.shape))


def inverse_broadcast_gradient(grad: OTensor, strides, shape, mode: str) -> OTensor:
    """grad/backwards.rs:516-538.  mode 'reference_literal' keeps only the *metadata* of `grad.sum_at(dim)` (line 527);
    mode 'sum' keeps the summed tensor, which is what the function's doc comment describes."""
    differential = grad.meta.rank() - len(shape)
    for dim, stride in enumerate(strides):
        if stride == 0:
            summed = grad.sum_at(dim)
            if mode == "sum":
                grad = summed
            else:
                grad = OTensor(grad.dtype, grad.buf, MetaTensor(list(summed.meta.shape), list(summed.meta.strides), summed.meta.offset), grad.is_view)
    for dim in range(len(strides) - 1, -1, -1):
        if strides[dim] == 0 and (dim < differential or shape[dim - differential] != 1):
            sq = grad.squeeze_at(dim)
            grad = OTensor(grad.dtype, grad.buf, sq.meta, grad.is_view)
    return grad


def train_step(x: OTensor, bias: OTensor, target: OTensor, lr: float, mode: str = "sum", seed_with_loss: bool = True):
    """One step of y = relu(x + bias), loss = mean_l1_loss(y, target), backward to d(bias), SGD, as the reference's engine
    sequences it (grad/mod.rs:432-495, grad/backwards.rs:7-42,148-161,229-239, grad/optim.rs:28-50).  `bias` is updated
    in place; returns (loss, d_bias)."""
    out_shape, stra, strb = compute_broadcasted_params(x.meta, bias.meta)
    pre = x + bias                                        # BroadcastAdd node
    y = pre.owned()
    gmap_relu = relu_grad_map(pre)                        # ReLU node
    y.unary_inplace("relu")
    loss, gmap_l1 = mean_l1_loss(y, target)               # L1 node
    upstream = loss.owned() if seed_with_loss else OTensor.from_buf(loss.dtype, [1], [])   # grad/mod.rs:442-447
    d_y = gmap_l1 * upstream                              # backwards_l1
    d_pre = gmap_relu * d_y                               # backwards_relu
    d_bias = inverse_broadcast_gradient(d_pre.owned(), strb, bias.meta.shape, mode)       # backwards_add, rhs
    grad = d_bias.owned() if not d_bias.is_view else d_bias                               # accumulate_grad: first assignment clones
    grad_values = OTensor(grad.dtype, cpu.gather(grad.dtype, grad.buf, grad.meta), MetaTensor.row_major(grad.meta.shape))
    update = grad_values * cpu.NP_DTYPE[grad.dtype].type(lr)                               # grad * lr
    v = bias.view()
    v -= update
    return loss, grad_values


def linear_step(x: OTensor, w: OTensor, target: OTensor, lr: float, seed_with_loss: bool = True):
    """One step of y = x @ w, loss = mean_l1_loss(y, target), backward to d(w), SGD (ops/linalg/matmul.rs:5-139, 182-198;
    backwards_matmul, grad/backwards.rs:493-510: d(rhs) = lhs^T @ upstream with only the last two dims swapped).  `w` is
    updated in place; returns (loss, d_w)."""
    y = x.matmul(w)                                       # MatMul node keeps contiguous copies of both inputs
    left = x.contiguous()
    loss, gmap_l1 = mean_l1_loss(y, target)               # L1 node
    upstream = loss.owned() if seed_with_loss else OTensor.from_buf(loss.dtype, [1], [])   # grad/mod.rs:442-447
    d_y = gmap_l1 * upstream                              # backwards_l1
    r = left.meta.rank()
    perm = list(range(r - 2)) + [r - 1, r - 2]
    d_w = left.permute(perm).matmul(d_y)                  # backwards_matmul, rhs
    update = d_w * cpu.NP_DTYPE[d_w.dtype].type(lr)
    v = w.view()
    v -= update
    return loss, d_w

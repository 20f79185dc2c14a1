"""Test helper: the reference's tensor surface (views, operators, reductions) driven through the C ABI of the HIP
backend.  Layout arithmetic comes from the oracle's metadata restatement, so a test can run the same program on the
oracle's OTensor and on a GTensor and compare buffers."""
from __future__ import annotations

import numpy as np

from oracle.meta import (MetaTensor, Slice, TensorError, compute_broadcasted_params, compute_permuted_parameters, contiguity_type,
                         compute_sliced_parameters, compute_squeezed_parameters, compute_unsqueezed_parameters, compute_view_as_parameters,
                         logical_to_buffer_idx, reduction_output_meta)
from rtensors_amd import hip as H


def _m(meta: MetaTensor):
    return (meta.offset, list(meta.shape), list(meta.strides))


# How the in-place unary / scalar / fill ops of a GTensor reach the backend:
#   "nd"         the whole (offset, shape, strides) through the `_nd` entry point (what the binding's dispatching methods do: the
#                library canonicalises the layout with signed strides)
#   "three_way"  the dispatch of the trait's default methods (backend/mod.rs:15-94): `_contiguous(offset, size)` when the view is
#                contiguous by the reference's |stride| rule (core/meta.rs:526-541), `_1d_strided(offset, stride, len)` when exactly one
#                dim is longer than 1, else `_nd` -- the three entry points as the reference's own code would call them
DISPATCH = "nd"


def _three_way(meta: MetaTensor):
    if meta.is_contiguous():
        return "contiguous", (meta.offset, meta.size())
    dims = meta.non_singleton_dims()
    if len(dims) == 1:
        _, size, stride = dims[0]
        return "1d_strided", (meta.offset, stride, size)
    return "nd", _m(meta)


class GTensor:
    def __init__(self, backend, buf, meta: MetaTensor, is_view=False):
        self.backend, self.buf, self.meta, self.is_view = backend, buf, meta, is_view
        self.dtype = buf.dtype

    @staticmethod
    def from_buf(backend, dtype, values, shape):
        if isinstance(dtype, str):
            dtype = H.DTYPE_BY_NAME[dtype]
        arr = np.asarray(values).astype(H.NP_DTYPE[dtype]).reshape(-1)
        meta = MetaTensor.row_major(list(shape))
        if arr.size != meta.size():
            raise TensorError("InvalidShape", "size")
        return GTensor(backend, backend.alloc_from_slice(dtype, arr), meta)

    def _view(self, shape, strides, offset):
        return GTensor(self.backend, self.buf, MetaTensor(list(shape), list(strides), offset), True)

    def view(self): return self._view(self.meta.shape, self.meta.strides, self.meta.offset)

    def slice(self, dim, sl):
        if isinstance(sl, int):
            sl = Slice.index(sl)
        return self._view(*compute_sliced_parameters(self.meta.shape, self.meta.strides, self.meta.offset, dim, sl))

    def permute(self, dims):
        shape, strides = compute_permuted_parameters(self.meta.shape, self.meta.strides, list(dims))
        return self._view(shape, strides, self.meta.offset)

    def transpose(self): return self.permute(list(range(self.meta.rank() - 1, -1, -1)))

    def unsqueeze_at(self, d):
        shape, strides = compute_unsqueezed_parameters(self.meta.shape, self.meta.strides, d)
        return self._view(shape, strides, self.meta.offset)

    def squeeze_at(self, d):
        shape, strides = compute_squeezed_parameters(self.meta.shape, self.meta.strides, d)
        return self._view(shape, strides, self.meta.offset)

    def squeeze(self):
        shape, strides = compute_squeezed_parameters(self.meta.shape, self.meta.strides, None)
        return self._view(shape, strides, self.meta.offset)

    def view_as(self, shape):
        return self._view(*compute_view_as_parameters(self.meta, list(shape)))

    def reshape(self, shape):
        c = self.contiguous()
        sh, st, off = compute_view_as_parameters(c.meta, list(shape))
        return GTensor(c.backend, c.buf, MetaTensor(sh, st, off))

    def get(self, idx):
        return self.backend.read(self.buf, logical_to_buffer_idx(list(idx), self.meta.strides, self.meta.offset))

    def set(self, idx, value):
        self.backend.write(self.buf, logical_to_buffer_idx(list(idx), self.meta.strides, self.meta.offset), value)

    def dump(self): return self.backend.dump(self.buf)

    def owned(self):
        if not self.is_view:
            return GTensor(self.backend, self.backend.copy(self.buf), MetaTensor(list(self.meta.shape), list(self.meta.strides), self.meta.offset))
        return self._gathered()

    def contiguous(self):
        if not self.is_view and self.meta.is_contiguous():
            return self.owned()
        return self._gathered()

    def _gathered(self):
        out = self.backend.alloc_uninit(self.dtype, self.meta.size())
        self.backend.gather(self.buf, _m(self.meta), out)
        return GTensor(self.backend, out, MetaTensor.row_major(self.meta.shape))

    def to_numpy(self):
        return self._gathered().dump().reshape(self.meta.shape)

    def _binary(self, other, op):
        out_shape, stra, strb = compute_broadcasted_params(self.meta, other.meta)
        result = GTensor(self.backend, self.backend.alloc(self.dtype, int(np.prod(out_shape, dtype=np.int64)) if out_shape else 1),
                         MetaTensor.row_major(out_shape))
        self.backend.broadcast((self.buf, (self.meta.offset, out_shape, stra)), (other.buf, (other.meta.offset, out_shape, strb)),
                               (result.buf, _m(result.meta)), op)
        return result

    def _binary_assign(self, other, op):
        out_shape, stra, strb = compute_broadcasted_params(self.meta, other.meta)
        if list(self.meta.shape) != list(out_shape):
            raise TensorError("Panic", "incompatible shapes for in-place op")
        a = (self.meta.offset, out_shape, stra)
        self.backend.broadcast((self.buf, a), (other.buf, (other.meta.offset, out_shape, strb)), (self.buf, a), op)
        return self

    def _scalar_assign(self, v, op):
        if DISPATCH == "three_way":
            entry, args = _three_way(self.meta)
            getattr(self.backend, f"scalar_{entry}")(op, self.buf, v, *args)
            return self
        self.backend.scalar_apply(op, self.buf, v, _m(self.meta))
        return self

    def _d(self, o, op, assign):
        if isinstance(o, GTensor):
            return self._binary_assign(o, op) if assign else self._binary(o, op)
        return self._scalar_assign(o, op) if assign else self.owned()._scalar_assign(o, op)

    def __add__(self, o): return self._d(o, "add", False)
    def __sub__(self, o): return self._d(o, "sub", False)
    def __mul__(self, o): return self._d(o, "mul", False)
    def __truediv__(self, o): return self._d(o, "div", False)
    def __iadd__(self, o): return self._d(o, "add", True)
    def __isub__(self, o): return self._d(o, "sub", True)
    def __imul__(self, o): return self._d(o, "mul", True)
    def __itruediv__(self, o): return self._d(o, "div", True)

    def unary_inplace(self, op):
        if DISPATCH == "three_way":
            entry, args = _three_way(self.meta)
            getattr(self.backend, f"unary_{entry}")(op, self.buf, *args)
            self.last_path = entry
            return self
        self.backend.apply_unary(op, self.buf, _m(self.meta))
        return self

    def unary(self, op): return self.owned().unary_inplace(op)

    def scalar_op_inplace(self, op, v):
        return self._scalar_assign(v, op)

    def fill(self, v):
        if DISPATCH == "three_way":
            entry, args = _three_way(self.meta)
            getattr(self.backend, f"fill_{entry}")(self.buf, v, *args)
            return
        self.backend.fill(self.buf, v, _m(self.meta))

    def matmul(self, other):
        """ops/linalg/matmul.rs:5-139 over the C ABI's rt_matmul."""
        if self.meta.rank() < 2 or other.meta.rank() < 2:
            raise TensorError("InvalidShape", "matmul operands need rank >= 2")
        def prepared(t):
            return t.contiguous() if contiguity_type(t.meta) == "none" or any(s < 0 for s in t.meta.strides) else t
        l, r = prepared(self), prepared(other)
        if l.meta.rank() != r.meta.rank():
            raise TensorError("InvalidShape", "rank mismatch")
        batch = list(l.meta.shape[:-2])
        if batch != list(r.meta.shape[:-2]):
            raise TensorError("SizeMismatch", "batch dims")
        m, k, kr, n = l.meta.shape[-2], l.meta.shape[-1], r.meta.shape[-2], r.meta.shape[-1]
        if k != kr:
            raise TensorError("SizeMismatch", "inner dims")
        b = int(np.prod(batch, dtype=np.int64)) if batch else 1
        om = MetaTensor.row_major(batch + [m, n])
        out = self.backend.alloc_uninit(self.dtype, max(om.size(), 1))
        self.backend.matmul((l.buf, _m(l.meta), contiguity_type(l.meta)), (r.buf, _m(r.meta), contiguity_type(r.meta)), out, b, m, k, n)
        return GTensor(self.backend, out, om)

    def dot(self, other):
        if self.meta.rank() != 1 or other.meta.rank() != 1:
            raise TensorError("InvalidShape", "Dot product is only defined for 1-D tensors")
        return self.unsqueeze_at(0).matmul(other.unsqueeze_at(1)).squeeze()

    def outer(self, other):
        if self.meta.rank() != 1 or other.meta.rank() != 1:
            raise TensorError("InvalidShape", "Outer product is only defined for 1-D tensors")
        return self.unsqueeze_at(1).matmul(other.unsqueeze_at(0))

    def reduce(self, op, axis=None):
        t = self if self.meta.is_contiguous() and all(s >= 0 for s in self.meta.strides) else self.contiguous()
        arg = op in ("argmax", "argmin")                          # do_argmax (ops/reduction/mod.rs:305-342): u64 output
        flat = self.backend.apply_argmax_contiguous_flat if arg else self.backend.apply_reduce_contiguous_flat
        nd = self.backend.apply_argmax_contiguous_nd if arg else self.backend.apply_reduce_contiguous_nd
        odt = H.U64 if arg else t.dtype
        if axis is None:
            out = self.backend.alloc(odt, 1)
            flat(t.buf, out, t.meta.offset, t.meta.size(), op)
            return GTensor(self.backend, out, MetaTensor([], [], 0))
        om = reduction_output_meta(t.meta, axis)
        out = self.backend.alloc(odt, om.size())
        if t.meta.rank() == 1:
            flat(t.buf, out, t.meta.offset, t.meta.size(), op)
        else:
            nd((t.buf, _m(t.meta)), out, axis, op)
        return GTensor(self.backend, out, om)

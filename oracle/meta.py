"""TEST INFRASTRUCTURE ONLY -- never imported by the product path.

Python restatement of the reference's host-side metadata arithmetic (pure integer bookkeeping, no tensor data).
Paths are relative to libs/rtensors/src/ of the reference.

Pinned by tests/test_oracle_meta.py against the reference's own expectations for slices, permutes, unsqueezes,
squeezes and broadcasting (core/mod.rs, core/slice.rs, ops/mod.rs test modules).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple


class TensorError(Exception):
    """Mirror of `TensorError` (core/tensor.rs:11-53); `kind` is the variant name."""

    def __init__(self, kind: str, msg: str = ""):
        super().__init__(f"{kind}: {msg}")
        self.kind = kind


def shape_to_stride(shape: Sequence[int]) -> List[int]:
    """core/meta.rs:495-503: row-major strides, last dim has stride 1."""
    stride = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        stride[i] = stride[i + 1] * shape[i + 1]
    return stride


@dataclass
class MetaTensor:
    """core/meta.rs:155-159."""

    shape: List[int]
    strides: List[int]
    offset: int = 0

    @staticmethod
    def row_major(shape: Sequence[int]) -> "MetaTensor":
        return MetaTensor(list(shape), shape_to_stride(shape), 0)

    def rank(self) -> int:
        return len(self.shape)

    def size(self) -> int:
        """core/meta.rs:186 (empty product = 1 for rank 0)."""
        n = 1
        for d in self.shape:
            n *= d
        return n

    def is_contiguous(self) -> bool:
        """core/meta.rs:526-541 (is_contiguous_relaxed): compares |stride|, skips size-1 dims."""
        if len(self.shape) == 0:
            return True
        if 0 in self.shape:
            return True
        if len(self.shape) != len(self.strides):
            return False
        expected = 1
        for dim, s in zip(reversed(self.shape), reversed(self.strides)):
            if dim != 1:
                if abs(s) != expected:
                    return False
                expected *= dim
        return True

    def is_flat(self) -> bool:
        """core/meta.rs:543-561: contiguity that allows an innermost |stride| other than 1 (used for matmul batch dims)."""
        if len(self.shape) == 0 or 0 in self.shape:
            return True
        if len(self.shape) != len(self.strides):
            return False
        expected = abs(self.strides[-1])
        for dim, s in zip(reversed(self.shape), reversed(self.strides)):
            if dim != 1:
                if abs(s) != expected:
                    return False
                expected *= dim
        return True

    def non_singleton_dims(self) -> List[Tuple[int, int, int]]:
        """core/meta.rs:618-625: (index, size, stride) of dims with size > 1."""
        return [(i, d, s) for i, (d, s) in enumerate(zip(self.shape, self.strides)) if d > 1]

    def inner_dimensions(self, dim: int) -> int:
        """core/meta.rs:209-218."""
        count = 1
        for i in range(dim + 1, len(self.shape)):
            count *= self.shape[i]
        return max(count, 1)

    def outer_dimensions(self, dim: int) -> int:
        """core/meta.rs:220-235."""
        count = 1
        for i in range(dim):
            count *= self.shape[i]
        return count

    def ith_offset(self, i: int) -> int:
        """core/meta.rs:310-326: buffer offset of the i-th element in row-major order."""
        idx = i
        off = self.offset
        for d in range(self.rank() - 1, -1, -1):
            dim = self.shape[d]
            off += (idx % dim) * self.strides[d]
            idx //= dim
        return off

    def dispatch(self) -> Tuple[str, tuple]:
        """backend/mod.rs:15-213, 239-268: the layout the default trait methods hand to the backend."""
        if self.is_contiguous():
            return "contiguous", (self.offset, self.size())
        nsd = self.non_singleton_dims()
        if len(nsd) == 1:
            _, dim_size, dim_stride = nsd[0]
            return "1d_strided", (self.offset, dim_stride, dim_size)
        return "nd", (self.offset, list(self.shape), list(self.strides))


@dataclass
class Slice:
    """core/slice.rs:17-52."""

    start: Optional[int] = None
    end: Optional[int] = None
    step: int = 1

    @staticmethod
    def full() -> "Slice":
        return Slice(None, None, 1)

    @staticmethod
    def index(i: int) -> "Slice":
        """`From<usize>` (core/slice.rs:107-115): start == end, which collapses the dim."""
        return Slice(i, i, 1)

    @staticmethod
    def range(a: int, b: int) -> "Slice":
        """`From<Range<usize>>` (core/slice.rs:54-63): a > b selects step -1."""
        return Slice(a, b, -1 if a > b else 1)

    @staticmethod
    def range_inclusive(a: int, b: int) -> "Slice":
        """`From<RangeInclusive<usize>>` (core/slice.rs:65-79)."""
        step = -1 if a > b else 1
        if step < 0:
            end = b - 1 if b > 0 else None
        else:
            end = b + 1
        return Slice(a, end, step)


def compute_sliced_parameters(shape, strides, offset, dim, sl: Slice):
    """core/slice.rs:145-239."""
    if dim >= len(shape):
        raise TensorError("InvalidDim", f"dimension {dim} out of bounds for rank {len(shape)}")
    step = sl.step
    if step == 0:
        raise TensorError("InvalidShape", "slice step cannot be zero")
    n = shape[dim]
    start = sl.start if sl.start is not None else (0 if step > 0 else n - 1)
    end = sl.end if sl.end is not None else (n if step > 0 else -1)
    if step > 0 and (start < 0 or start >= n or end < 0 or end > n):
        raise TensorError("IdxOutOfBounds", f"slice {start}..{end} out of bounds for size {n}")
    if step < 0 and (start < 0 or start >= n or end < -1 or end >= n):
        raise TensorError("IdxOutOfBounds", f"slice {start}..{end} out of bounds for size {n}")
    if (step > 0 and start >= end) or (step < 0 and start <= end):
        length = 0
    else:
        length = (abs(start - end) - 1) // abs(step) + 1
    new_offset = offset + max(start * strides[dim], 0)
    new_shape = list(shape)
    new_strides = list(strides)
    if length == 0:
        del new_shape[dim]
        del new_strides[dim]
        return new_shape, new_strides, new_offset
    new_shape[dim] = length
    new_strides[dim] = strides[dim] * step
    return new_shape, new_strides, new_offset


def compute_permuted_parameters(shape, strides, dims):
    """core/tensor.rs:909-941."""
    rank = len(shape)
    if len(dims) != rank:
        raise TensorError("WrongDims", f"permutation of length {len(dims)} for rank {rank}")
    for d in dims:
        if d >= rank:
            raise TensorError("InvalidDim", f"permutation dim {d} out of bounds for rank {rank}")
    return [shape[d] for d in dims], [strides[d] for d in dims]


def compute_unsqueezed_parameters(shape, strides, dim):
    """core/tensor.rs:973-990: the inserted dim gets stride `stride[dim] * shape[dim]` (1 * 1 past the end)."""
    if dim > len(shape):
        raise TensorError("InvalidDim", f"unsqueeze dim {dim} out of bounds for rank {len(shape)}")
    lstr = strides[dim] if dim < len(strides) else 1
    lsh = shape[dim] if dim < len(shape) else 1
    new_shape = list(shape)
    new_strides = list(strides)
    new_strides.insert(dim, lstr * lsh)
    new_shape.insert(dim, 1)
    return new_shape, new_strides


def compute_squeezed_parameters(shape, strides, dim: Optional[int]):
    """core/tensor.rs:993-1027."""
    if dim is not None and dim >= len(shape):
        raise TensorError("InvalidDim", f"dimension {dim} out of bounds for rank {len(shape)}")
    new_shape = list(shape)
    new_strides = list(strides)
    for d in range(len(shape) - 1, -1, -1):
        should = (shape[d] == 1) if dim is None else (dim == d)
        if should:
            if shape[d] != 1:
                raise TensorError("InvalidDim", f"cannot squeeze dimension {d} with size {shape[d]}")
            del new_shape[d]
            del new_strides[d]
    return new_shape, new_strides


def compute_view_as_parameters(meta: "MetaTensor", new_shape):
    """core/tensor.rs:328-355 (`view_as_inner`): the layout must pass the relaxed contiguity check and the element counts must agree;
    the result has the new shape's row-major strides and the same offset (whatever the signs of the old strides were)."""
    if not meta.is_contiguous():
        raise TensorError("ContiguityError", "cannot view_as a non-contiguous tensor")
    n = 1
    for d in new_shape:
        n *= d
    if n != meta.size():
        raise TensorError("InvalidShape", f"invalid size {n} for initial size {meta.size()}")
    return list(new_shape), shape_to_stride(list(new_shape)), meta.offset


def compute_broadcasted_params(a: MetaTensor, b: MetaTensor):
    """ops/broadcast/mod.rs:13-55: (out_shape, a_strides, b_strides)."""
    sa, sb = list(a.shape), list(b.shape)
    stra, strb = list(a.strides), list(b.strides)
    if len(sa) < len(sb):
        pad = len(sb) - len(sa)
        sa = [1] * pad + sa
        stra = [0] * pad + stra
    if len(sb) < len(sa):
        pad = len(sa) - len(sb)
        sb = [1] * pad + sb
        strb = [0] * pad + strb
    out_shape, out_stra, out_strb = [], [], []
    for i in range(len(sa)):
        x, y = sa[i], sb[i]
        if x == y:
            out = x
        elif x == 1:
            out = y
        elif y == 1:
            out = x
        else:
            raise TensorError("BroadcastError", f"shapes {sa} and {sb} are not broadcastable")
        out_shape.append(out)
        out_stra.append(0 if (x == 1 and out > 1) else stra[i])
        out_strb.append(0 if (y == 1 and out > 1) else strb[i])
    return out_shape, out_stra, out_strb


def reduction_output_meta(inp: MetaTensor, axis: Optional[int]) -> MetaTensor:
    """ops/reduction/mod.rs:512-538 (axis) and 276-277 (`Idx::Item` -> rank 0)."""
    if axis is None:
        return MetaTensor([], [], 0)
    shape = [1 if d == axis else inp.shape[d] for d in range(inp.rank())]
    return MetaTensor(shape, shape_to_stride(shape), 0)


def logical_to_buffer_idx(idx: Sequence[int], strides: Sequence[int], offset: int) -> int:
    """core/tensor.rs:871-906."""
    if len(idx) != len(strides):
        raise TensorError("WrongDims", f"index rank {len(idx)} does not match tensor rank {len(strides)}")
    b = offset
    for i, s in zip(idx, strides):
        b += i * s
    if b < 0:
        raise TensorError("IdxOutOfBounds", "buffer index is negative")
    return b


def contiguity_type(meta: MetaTensor) -> str:
    """ops/linalg/matmul.rs:200-251: layout of the last two dims as gemm sees it ("row_major": last stride 1; "column_major":
    second-to-last stride 1; else "none"), "none" as well when several batch dims do not collapse into one stride."""
    r = meta.rank()
    if r < 2:
        return "row_major"
    if meta.strides[r - 1] == 1:
        inner = "row_major"
    elif meta.strides[r - 2] == 1:
        inner = "column_major"
    else:
        inner = "none"
    batch = MetaTensor(list(meta.shape[:r - 2]), list(meta.strides[:r - 2]), 0)
    if batch.rank() > 1 and not batch.is_flat():
        return "none"
    return inner


def view_bounds(offset: int, shape: Sequence[int], strides: Sequence[int]) -> Tuple[int, int]:
    """Lowest and highest buffer index a non-empty view addresses (exact integers)."""
    lo = hi = offset
    for d, s in zip(shape, strides):
        span = (d - 1) * s
        if span < 0:
            lo += span
        else:
            hi += span
    return lo, hi


def check_extent(offset: int, shape: Sequence[int], strides: Sequence[int], length: int) -> Tuple[str, int]:
    """`check_extent` of the reference's remote server (backend/remote/server.rs:241-275): ("ok", element count), ("invalid", 0) for a
    malformed descriptor, ("out_of_bounds", 0) when an addressed element lies outside [0, length).  The element count is folded left
    to right with `checked_mul` over usize, so an overflow met before a zero dim is an error.  Two rules are tighter than the
    reference's: a buffer length or a non-empty view's element count beyond i64::MAX is refused (device kernels index with signed
    64-bit integers)."""
    if len(shape) != len(strides) or length > (1 << 63) - 1:
        return "invalid", 0
    n = 1
    for d in shape:
        n *= d
        if n > (1 << 64) - 1:
            return "invalid", 0
    if any(d == 0 for d in shape):
        return ("out_of_bounds", 0) if offset > length else ("ok", 0)
    if n > (1 << 63) - 1:
        return "invalid", 0
    lo, hi = view_bounds(offset, shape, strides)
    if lo < 0 or hi >= length:
        return "out_of_bounds", 0
    return "ok", n

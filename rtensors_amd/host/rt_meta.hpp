// Host-side tensor metadata: shapes, signed strides, offsets and the view arithmetic of the reference
// (libs/rtensors/src/core/meta.rs, core/slice.rs, core/tensor.rs, ops/broadcast/mod.rs, ops/reduction/mod.rs).
// Pure integer bookkeeping; nothing here touches a device.
#pragma once

#include <cstdint>
#include <cstdlib>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace rt {

// TensorError (core/tensor.rs:11-53); HipError stands where the cfg-gated CudaError stands.
enum class ErrorKind {
    InvalidShape, InvalidDim, IdxOutOfBounds, WrongDims, BroadcastError, SizeMismatch, UnsupportedOperation, GradError, HipError,
    Panic,  // where the reference's operator sugar unwraps / panics (e.g. in-place op that would have to grow the lhs)
    ContiguityError
};

inline const char* kind_name(ErrorKind k) {
    switch (k) {
        case ErrorKind::InvalidShape: return "InvalidShape";
        case ErrorKind::InvalidDim: return "InvalidDim";
        case ErrorKind::IdxOutOfBounds: return "IdxOutOfBounds";
        case ErrorKind::WrongDims: return "WrongDims";
        case ErrorKind::BroadcastError: return "BroadcastError";
        case ErrorKind::SizeMismatch: return "SizeMismatch";
        case ErrorKind::UnsupportedOperation: return "UnsupportedOperation";
        case ErrorKind::GradError: return "GradError";
        case ErrorKind::HipError: return "HipError";
        case ErrorKind::Panic: return "Panic";
        case ErrorKind::ContiguityError: return "ContiguityError";
    }
    return "?";
}

struct TensorError : std::runtime_error {
    ErrorKind kind;
    TensorError(ErrorKind k, const std::string& msg) : std::runtime_error(std::string(kind_name(k)) + ": " + msg), kind(k) {}
};

using Shape = std::vector<uint64_t>;
using Strides = std::vector<int64_t>;

// core/meta.rs:495-503
inline Strides shape_to_stride(const Shape& shape) {
    Strides st(shape.size(), 1);
    for (size_t i = shape.size(); i-- > 0;)
        if (i + 1 < shape.size()) st[i] = st[i + 1] * (int64_t)shape[i + 1];
    return st;
}

// core/slice.rs:17-52 and the From<Range..> conversions at 54-115
struct Slice {
    std::optional<uint64_t> start, end;
    int64_t step = 1;
    static Slice full() { return Slice{std::nullopt, std::nullopt, 1}; }
    static Slice index(uint64_t i) { return Slice{i, i, 1}; }                                   // From<usize>
    static Slice range(uint64_t a, uint64_t b) { return Slice{a, b, a > b ? -1 : 1}; }          // From<Range<usize>>
    static Slice range_inclusive(uint64_t a, uint64_t b) {                                      // From<RangeInclusive<usize>>
        int64_t step = a > b ? -1 : 1;
        if (step < 0) return Slice{a, b > 0 ? std::optional<uint64_t>(b - 1) : std::nullopt, step};
        return Slice{a, b + 1, step};
    }
    Slice with_step(int64_t s) const { Slice r = *this; r.step = s; return r; }
};

struct NonSingleton { size_t dim; uint64_t size; int64_t stride; };

// core/meta.rs:155-159
struct MetaTensor {
    Shape shape;
    Strides strides;
    uint64_t offset = 0;

    MetaTensor() = default;
    MetaTensor(Shape s, Strides st, uint64_t off) : shape(std::move(s)), strides(std::move(st)), offset(off) {}
    static MetaTensor row_major(const Shape& s) { return MetaTensor(s, shape_to_stride(s), 0); }

    size_t rank() const { return shape.size(); }
    uint64_t size() const { uint64_t n = 1; for (uint64_t d : shape) n *= d; return n; }          // core/meta.rs:186
    bool is_scalar() const { return strides.empty(); }

    // core/meta.rs:526-541 (is_contiguous_relaxed).  Compares |stride|: a fully reversed view counts as contiguous.
    bool is_contiguous() const {
        if (shape.empty()) return true;
        for (uint64_t d : shape) if (d == 0) return true;
        if (shape.size() != strides.size()) return false;
        uint64_t expected = 1;
        for (size_t i = shape.size(); i-- > 0;) {
            if (shape[i] != 1) {
                uint64_t a = strides[i] < 0 ? (uint64_t)(-(strides[i] + 1)) + 1 : (uint64_t)strides[i];
                if (a != expected) return false;
                uint64_t p;
                expected = __builtin_mul_overflow(expected, shape[i], &p) ? UINT64_MAX : p;
            }
        }
        return true;
    }
    // core/meta.rs:543-561: contiguity that allows an innermost |stride| other than 1 (matmul batch dims)
    bool is_flat() const {
        if (shape.empty()) return true;
        for (uint64_t d : shape) if (d == 0) return true;
        if (shape.size() != strides.size()) return false;
        auto mag = [](int64_t s) { return s < 0 ? (uint64_t)(-(s + 1)) + 1 : (uint64_t)s; };
        uint64_t expected = mag(strides.back());
        for (size_t i = shape.size(); i-- > 0;) {
            if (shape[i] != 1) {
                if (mag(strides[i]) != expected) return false;
                uint64_t p;
                expected = __builtin_mul_overflow(expected, shape[i], &p) ? UINT64_MAX : p;
            }
        }
        return true;
    }
    // Forward row-major run: what a kernel may treat as `offset .. offset + size` (signed strides).
    bool is_forward_contiguous() const {
        int64_t expected = 1;
        for (size_t i = shape.size(); i-- > 0;) {
            if (shape[i] == 0) return true;
            if (shape[i] != 1) {
                if (strides[i] != expected) return false;
                expected *= (int64_t)shape[i];
            }
        }
        return true;
    }
    // core/meta.rs:618-625
    std::vector<NonSingleton> non_singleton_dims() const {
        std::vector<NonSingleton> out;
        for (size_t i = 0; i < shape.size(); ++i) if (shape[i] > 1) out.push_back({i, shape[i], strides[i]});
        return out;
    }
    // core/meta.rs:209-235
    uint64_t inner_dimensions(size_t dim) const {
        uint64_t c = 1;
        for (size_t i = dim + 1; i < shape.size(); ++i) c *= shape[i];
        return c < 1 ? 1 : c;
    }
    uint64_t outer_dimensions(size_t dim) const {
        uint64_t c = 1;
        for (size_t i = 0; i < dim; ++i) c *= shape[i];
        return c;
    }
    // core/meta.rs:310-326
    uint64_t ith_offset(uint64_t i) const {
        int64_t off = (int64_t)offset;
        for (size_t d = shape.size(); d-- > 0;) {
            off += (int64_t)(i % shape[d]) * strides[d];
            i /= shape[d];
        }
        return (uint64_t)off;
    }
};

// core/tensor.rs:871-906
inline uint64_t logical_to_buffer_idx(const std::vector<uint64_t>& idx, const Strides& strides, uint64_t offset) {
    if (idx.size() != strides.size())
        throw TensorError(ErrorKind::WrongDims, "Index rank " + std::to_string(idx.size()) + " does not match tensor rank " + std::to_string(strides.size()));
    int64_t b = (int64_t)offset;
    for (size_t i = 0; i < idx.size(); ++i) b += (int64_t)idx[i] * strides[i];
    if (b < 0) throw TensorError(ErrorKind::IdxOutOfBounds, "Buffer index is negative");
    return (uint64_t)b;
}

// core/slice.rs:145-239
inline MetaTensor compute_sliced_parameters(const MetaTensor& m, size_t dim, const Slice& sl) {
    if (dim >= m.shape.size())
        throw TensorError(ErrorKind::InvalidDim, "Dimension " + std::to_string(dim) + " out of bounds for shape with rank " + std::to_string(m.shape.size()));
    const int64_t step = sl.step;
    if (step == 0) throw TensorError(ErrorKind::InvalidShape, "Slice step cannot be zero");
    const int64_t n = (int64_t)m.shape[dim];
    const int64_t start = sl.start ? (int64_t)*sl.start : (step > 0 ? 0 : n - 1);
    const int64_t end = sl.end ? (int64_t)*sl.end : (step > 0 ? n : -1);
    if ((step > 0 && (start < 0 || start >= n || end < 0 || end > n)) || (step < 0 && (start < 0 || start >= n || end < -1 || end >= n)))
        throw TensorError(ErrorKind::IdxOutOfBounds, "Slice indices out of bounds for dimension " + std::to_string(dim) + " with size " +
                                                         std::to_string(n) + ": start " + std::to_string(start) + ", end " + std::to_string(end));
    uint64_t len = 0;
    if (!((step > 0 && start >= end) || (step < 0 && start <= end)))
        len = (uint64_t)((std::llabs(start - end) - 1) / std::llabs(step)) + 1;
    const int64_t shift = start * m.strides[dim];
    MetaTensor out = m;
    out.offset = m.offset + (uint64_t)(shift > 0 ? shift : 0);
    if (len == 0) {                              // single index (start == end) or empty range: the dim disappears
        out.shape.erase(out.shape.begin() + (long)dim);
        out.strides.erase(out.strides.begin() + (long)dim);
        return out;
    }
    out.shape[dim] = len;
    out.strides[dim] = m.strides[dim] * step;
    return out;
}

// core/tensor.rs:909-941
inline MetaTensor compute_permuted_parameters(const MetaTensor& m, const std::vector<size_t>& dims) {
    const size_t rank = m.shape.size();
    if (dims.size() != rank)
        throw TensorError(ErrorKind::WrongDims, "Permutation dims length " + std::to_string(dims.size()) + " does not match tensor rank " + std::to_string(rank));
    MetaTensor out;
    out.offset = m.offset;
    for (size_t d : dims) {
        if (d >= rank) throw TensorError(ErrorKind::InvalidDim, "Permutation dim " + std::to_string(d) + " is out of bounds for tensor rank " + std::to_string(rank));
        out.shape.push_back(m.shape[d]);
        out.strides.push_back(m.strides[d]);
    }
    return out;
}

// core/tensor.rs:973-990: the new dim gets stride `stride[dim] * shape[dim]` (1 * 1 when appended at the end)
inline MetaTensor compute_unsqueezed_parameters(const MetaTensor& m, size_t dim) {
    if (dim > m.shape.size())
        throw TensorError(ErrorKind::InvalidDim, "Unsqueeze dim " + std::to_string(dim) + " is out of bounds for tensor rank " + std::to_string(m.shape.size()));
    MetaTensor out = m;
    const int64_t lstr = dim < m.strides.size() ? m.strides[dim] : 1;
    const int64_t lsh = dim < m.shape.size() ? (int64_t)m.shape[dim] : 1;
    out.strides.insert(out.strides.begin() + (long)dim, lstr * lsh);
    out.shape.insert(out.shape.begin() + (long)dim, 1);
    return out;
}

// core/tensor.rs:993-1027
inline MetaTensor compute_squeezed_parameters(const MetaTensor& m, std::optional<size_t> dim) {
    if (dim && *dim >= m.shape.size())
        throw TensorError(ErrorKind::InvalidDim, "Dimension " + std::to_string(*dim) + " is out of bounds for tensor with rank " + std::to_string(m.shape.size()));
    MetaTensor out = m;
    for (size_t d = m.shape.size(); d-- > 0;) {
        const bool should = dim ? (*dim == d) : (m.shape[d] == 1);
        if (!should) continue;
        if (m.shape[d] != 1)
            throw TensorError(ErrorKind::InvalidDim, "Cannot squeeze dimension " + std::to_string(d) + " with size " + std::to_string(m.shape[d]));
        out.shape.erase(out.shape.begin() + (long)d);
        out.strides.erase(out.strides.begin() + (long)d);
    }
    return out;
}

// core/tensor.rs:328-355 (`view_as_inner`): a layout that passes the relaxed contiguity check is given another shape of the same
// element count, with that shape's row-major strides and the same offset.  The reference does this whatever the signs of the old
// strides are, which for a reversed view (|stride| contiguous, offset at its first element = the run's last address) describes
// memory past the run.  Here a view whose non-singleton strides are all negative gets the negated row-major strides, so that
// element k of the new shape is still element k of the old one; mixed signs cannot be expressed by strides and are refused.
inline MetaTensor compute_view_as_parameters(const MetaTensor& m, const Shape& shape) {
    if (!m.is_contiguous()) throw TensorError(ErrorKind::ContiguityError, "Cannot view_as non contiguous tensor");
    uint64_t n = 1;
    for (uint64_t d : shape) n *= d;
    if (n != m.size()) throw TensorError(ErrorKind::InvalidShape, "Invalid size " + std::to_string(n) + " for initial shape " + std::to_string(m.size()));
    bool neg = false, pos = false;
    for (size_t d = 0; d < m.shape.size(); ++d)
        if (m.shape[d] > 1) (m.strides[d] < 0 ? neg : pos) = true;
    if (neg && pos && n > 0) throw TensorError(ErrorKind::ContiguityError, "Cannot view_as a view reversed along some of its dims only");
    MetaTensor out = MetaTensor::row_major(shape);
    out.offset = m.offset;
    if (neg) for (auto& st : out.strides) st = -st;
    return out;
}

struct BroadcastParams { Shape shape; Strides a, b; };

// ops/broadcast/mod.rs:13-55
inline BroadcastParams compute_broadcasted_params(const MetaTensor& a, const MetaTensor& b) {
    Shape sa = a.shape, sb = b.shape;
    Strides stra = a.strides, strb = b.strides;
    if (sa.size() < sb.size()) {
        size_t pad = sb.size() - sa.size();
        sa.insert(sa.begin(), pad, 1);
        stra.insert(stra.begin(), pad, 0);
    }
    if (sb.size() < sa.size()) {
        size_t pad = sa.size() - sb.size();
        sb.insert(sb.begin(), pad, 1);
        strb.insert(strb.begin(), pad, 0);
    }
    BroadcastParams out;
    for (size_t i = 0; i < sa.size(); ++i) {
        uint64_t x = sa[i], y = sb[i], o;
        if (x == y) o = x;
        else if (x == 1) o = y;
        else if (y == 1) o = x;
        else throw TensorError(ErrorKind::BroadcastError, "Shapes are not broadcastable");
        out.shape.push_back(o);
        out.a.push_back((x == 1 && o > 1) ? 0 : stra[i]);
        out.b.push_back((y == 1 && o > 1) ? 0 : strb[i]);
    }
    return out;
}

// ops/reduction/mod.rs:512-538 (axis kept with size 1) and 276-277 (full reduction -> rank 0)
inline MetaTensor reduction_output_meta(const MetaTensor& in, std::optional<size_t> axis) {
    if (!axis) return MetaTensor({}, {}, 0);
    Shape s;
    for (size_t d = 0; d < in.rank(); ++d) s.push_back(d == *axis ? 1 : in.shape[d]);
    return MetaTensor::row_major(s);
}

// core/meta.rs:744-750; codes equal rt_contiguity of the C ABI
enum class ContiguityTypes { RowMajor = 0, ColumnMajor = 1, None = 2 };

// ops/linalg/matmul.rs:200-251: the layout gemm sees in the last two dims; None as well when several batch dims do not
// collapse into one stride
inline ContiguityTypes contiguity_type(const MetaTensor& meta) {
    const size_t r = meta.rank();
    if (r < 2) return ContiguityTypes::RowMajor;
    ContiguityTypes inner = meta.strides[r - 1] == 1 ? ContiguityTypes::RowMajor
                          : meta.strides[r - 2] == 1 ? ContiguityTypes::ColumnMajor : ContiguityTypes::None;
    MetaTensor batch(Shape(meta.shape.begin(), meta.shape.end() - 2), Strides(meta.strides.begin(), meta.strides.end() - 2), 0);
    if (batch.rank() > 1 && !batch.is_flat()) return ContiguityTypes::None;
    return inner;
}

}  // namespace rt

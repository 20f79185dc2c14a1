// Tensors, views and operators on the Hip backend, following the reference's operator glue: which backend call each
// operator issues and with which (offset, shape, strides).
//   constructors / owned / contiguous : core/primitives.rs:68-123, 367-506; core/tensor.rs:215-325
//   views (pure metadata)             : core/tensor.rs:548-628
//   broadcast operators               : ops/broadcast/add.rs:7-478 (sub / mul / div are textual twins)
//   scalar operators                  : ops/scalar/add.rs:20-121
//   unary ops                         : ops/unary/mod.rs:56-126
//   reductions                        : ops/reduction/mod.rs:262-302, 346-408
// `Tensor` carries its dtype at run time (the reference resolves `T` at run time too, via TypeId, backend/cuda.rs:221-231);
// `TensorBase<T>` is the typed face of it.  A Tensor with `is_view()` shares its buffer with the tensor it came from,
// like TensorView / TensorViewMut.
#pragma once

#include <optional>
#include <vector>

#include "rt_backend.hpp"

namespace rt {

class Tensor {
  public:
    Tensor() = default;
    Tensor(Hip backend, Buf buf, MetaTensor meta, bool is_view = false)
        : backend_(std::make_shared<Hip>(std::move(backend))), buf_(std::move(buf)), meta_(std::move(meta)), is_view_(is_view) {}

    // ---- constructors -------------------------------------------------------------------------------------------------
    // TensorBase::from_buf (core/primitives.rs:367-400): row-major, offset 0; length must match the shape.
    static Tensor from_buf(const Hip& backend, int dtype, const void* host, uint64_t len, const Shape& shape) {
        MetaTensor m = MetaTensor::row_major(shape);
        if (m.size() != len) throw TensorError(ErrorKind::InvalidShape, "Element count does not match shape");
        return Tensor(backend, backend.alloc_from_slice(dtype, host, len), m);
    }
    // zeros / ones / full on the device: a fill kernel, not the host Vec + upload of core/primitives.rs:455-506
    static Tensor full(const Hip& backend, int dtype, const Shape& shape, const Scalar& v) {
        MetaTensor m = MetaTensor::row_major(shape);
        Buf b = backend.alloc_uninit(dtype, m.size());
        backend.fill_contiguous(*b, v, 0, m.size());
        return Tensor(backend, b, m);
    }
    static Tensor zeros(const Hip& backend, int dtype, const Shape& shape) {
        MetaTensor m = MetaTensor::row_major(shape);
        return Tensor(backend, backend.alloc(dtype, m.size()), m);
    }
    static Tensor ones(const Hip& backend, int dtype, const Shape& shape) { return full(backend, dtype, shape, Scalar::from_double(dtype, 1.0)); }
    // TensorBase::max / ::min (core/primitives.rs:490-506): every element T::MAX / T::MIN, filled on the device
    static Tensor max(const Hip& backend, int dtype, const Shape& shape) { return full(backend, dtype, shape, Scalar::limit(dtype, true)); }
    static Tensor min(const Hip& backend, int dtype, const Shape& shape) { return full(backend, dtype, shape, Scalar::limit(dtype, false)); }
    // TensorBase::scalar / ::column / ::row (core/primitives.rs:418-444): shapes [], [n] and [1, n]
    static Tensor scalar(const Hip& backend, const Scalar& v) { return from_buf(backend, v.dtype, v.bytes, 1, Shape{}); }
    static Tensor column(const Hip& backend, int dtype, const void* host, uint64_t n) { return from_buf(backend, dtype, host, n, Shape{n}); }
    static Tensor row(const Hip& backend, int dtype, const void* host, uint64_t n) { return from_buf(backend, dtype, host, n, Shape{1, n}); }
    // TensorBase::into_dtype (core/primitives.rs:527-539): a new buffer of meta.size() elements of the other type, the whole
    // source buffer converted into it (SizeMismatch when the two lengths differ, as for a view of part of a buffer), same meta
    Tensor into_dtype(int new_dtype) const {
        Buf nb = backend_->alloc_uninit(new_dtype, meta_.size());
        backend_->convert(*buf_, *nb);
        return Tensor(*backend_, nb, meta_);
    }

    // ---- accessors ------------------------------------------------------------------------------------------------------
    const MetaTensor& meta() const { return meta_; }
    const Shape& shape() const { return meta_.shape; }
    const Strides& strides() const { return meta_.strides; }
    uint64_t offset() const { return meta_.offset; }
    uint64_t size() const { return meta_.size(); }
    size_t rank() const { return meta_.rank(); }
    bool is_contiguous() const { return meta_.is_contiguous(); }
    bool is_view() const { return is_view_; }
    int dtype() const { return buf_->dtype(); }
    const Hip& backend() const { return *backend_; }
    const Buf& buf() const { return buf_; }

    // ---- views: metadata only --------------------------------------------------------------------------------------------
    Tensor view() const { return with_meta(meta_); }
    Tensor slice(size_t dim, const Slice& s) const { return with_meta(compute_sliced_parameters(meta_, dim, s)); }
    Tensor permute(const std::vector<size_t>& dims) const { return with_meta(compute_permuted_parameters(meta_, dims)); }
    Tensor transpose() const {
        std::vector<size_t> d(rank());
        for (size_t i = 0; i < d.size(); ++i) d[i] = d.size() - 1 - i;
        return permute(d);
    }
    Tensor unsqueeze_at(size_t dim) const { return with_meta(compute_unsqueezed_parameters(meta_, dim)); }
    Tensor squeeze_at(size_t dim) const { return with_meta(compute_squeezed_parameters(meta_, dim)); }
    Tensor squeeze() const { return with_meta(compute_squeezed_parameters(meta_, std::nullopt)); }
    // TensorAccess::slice_at / ::unsqueeze (core/tensor.rs:443-445, 462-464)
    Tensor slice_at(size_t dim, uint64_t at) const { return slice(dim, Slice::index(at)); }
    Tensor unsqueeze() const { return unsqueeze_at(0); }
    // the in-place metadata forms of an owner (core/primitives.rs:509-524)
    void squeeze_inplace() { meta_ = compute_squeezed_parameters(meta_, std::nullopt); }
    void unsqueeze_at_inplace(size_t dim) { meta_ = compute_unsqueezed_parameters(meta_, dim); }
    void unsqueeze_inplace() { unsqueeze_at_inplace(0); }

    // ---- element access (core/tensor.rs:535-541, 665-688) ----------------------------------------------------------------------
    Scalar get(const std::vector<uint64_t>& idx) const { return backend_->read(*buf_, logical_to_buffer_idx(idx, meta_.strides, meta_.offset)); }
    void set(const std::vector<uint64_t>& idx, const Scalar& v) { backend_->write(*buf_, logical_to_buffer_idx(idx, meta_.strides, meta_.offset), v); }
    Scalar item() const {
        if (size() != 1) throw TensorError(ErrorKind::WrongDims, "item() needs a single-element tensor");
        return backend_->read(*buf_, meta_.ith_offset(0));
    }
    void fill(const Scalar& v) { backend_->fill(*buf_, v, meta_); }

    // Would owned() give a row-major tensor holding exactly this tensor's elements in order?  Then `op(owned())` can be
    // computed in one pass from this tensor's run into a fresh buffer.  A view: whenever it is a forward contiguous run
    // (owned() gathers it).  An owner: only when its buffer is that run and nothing else (owned() clones the whole buffer
    // and keeps the meta).
    bool one_pass_ok() const {
        if (size() == 0 || !meta_.is_forward_contiguous()) return false;
        if (is_view_) return true;
        return meta_.offset == 0 && buf_->len() == size() && meta_.strides == shape_to_stride(meta_.shape);
    }
    Tensor like_row_major() const { return Tensor(*backend_, backend_->alloc_uninit(dtype(), size()), MetaTensor::row_major(meta_.shape)); }

    // ---- owned / contiguous -------------------------------------------------------------------------------------------------------
    // TensorBase::owned = Clone: the whole buffer, same meta.  A view's owned() gathers into a fresh row-major buffer.
    Tensor owned() const {
        if (!is_view_) return Tensor(*backend_, backend_->copy(*buf_), meta_);
        return gathered();
    }
    Tensor contiguous() const {
        if (!is_view_ && meta_.is_contiguous()) return owned();
        return gathered();
    }
    // `.cpu()` (core/primitives.rs:104-112) downloads the whole underlying buffer and keeps the meta; this returns the
    // elements the tensor addresses, row-major, which is what a caller compares against.
    void to_host(void* dst) const {
        Tensor g = gathered();
        backend_->dump(*g.buf_, dst);
    }
    void dump_buffer(void* dst) const { backend_->dump(*buf_, dst); }

    // ---- broadcast operators -----------------------------------------------------------------------------------------------------------
    Tensor binary(const Tensor& rhs, BinaryOpType op) const {
        BroadcastParams p = compute_broadcasted_params(meta_, rhs.meta_);
        MetaTensor out = MetaTensor::row_major(p.shape);
        // the reference zero-fills the result (zeros_on, add.rs:185); every element is overwritten, so skip the fill
        Tensor result(*backend_, backend_->alloc_uninit(dtype(), out.size()), out);
        backend_->broadcast(*buf_, MetaTensor(p.shape, p.a, meta_.offset), *rhs.buf_, MetaTensor(p.shape, p.b, rhs.meta_.offset), *result.buf_, out, op);
        return result;
    }
    Tensor& binary_assign(const Tensor& rhs, BinaryOpType op) {
        BroadcastParams p = compute_broadcasted_params(meta_, rhs.meta_);
        if (meta_.shape != p.shape) throw TensorError(ErrorKind::Panic, "Incompatible shapes for in-place operation: rhs does not broadcast to lhs");
        MetaTensor a(p.shape, p.a, meta_.offset);
        backend_->broadcast(*buf_, a, *rhs.buf_, MetaTensor(p.shape, p.b, rhs.meta_.offset), *buf_, a, op);
        return *this;
    }
    Tensor operator+(const Tensor& o) const { return binary(o, BinaryOpType::Add); }
    Tensor operator-(const Tensor& o) const { return binary(o, BinaryOpType::Sub); }
    Tensor operator*(const Tensor& o) const { return binary(o, BinaryOpType::Mul); }
    Tensor operator/(const Tensor& o) const { return binary(o, BinaryOpType::Div); }
    Tensor& operator+=(const Tensor& o) { return binary_assign(o, BinaryOpType::Add); }
    Tensor& operator-=(const Tensor& o) { return binary_assign(o, BinaryOpType::Sub); }
    Tensor& operator*=(const Tensor& o) { return binary_assign(o, BinaryOpType::Mul); }
    Tensor& operator/=(const Tensor& o) { return binary_assign(o, BinaryOpType::Div); }

    // ---- scalar operators: `t op= s` is one in-place kernel; `t op s` is owned() + in-place in the reference
    // (ops/scalar/add.rs:84-113), here one out-of-place pass when the operand is a forward contiguous run -----------------------------
    Tensor& scalar_assign(int op, const Scalar& v) { backend_->scalar_apply(op, *buf_, v, meta_); return *this; }
    Tensor scalar(int op, const Scalar& v) const {
        if (one_pass_ok()) {
            Tensor r = like_row_major();
            backend_->scalar_apply_to(op, *buf_, v, meta_.offset, size(), *r.buf_);
            return r;
        }
        Tensor r = owned();
        r.scalar_assign(op, v);
        return r;
    }
    Tensor& scalar_assign(int op, double v) { return scalar_assign(op, Scalar::from_double(dtype(), v)); }
    Tensor scalar(int op, double v) const { return scalar(op, Scalar::from_double(dtype(), v)); }
    Tensor operator+(double s) const { return scalar(RT_S_ADD, s); }
    Tensor operator-(double s) const { return scalar(RT_S_SUB, s); }
    Tensor operator*(double s) const { return scalar(RT_S_MUL, s); }
    Tensor operator/(double s) const { return scalar(RT_S_DIV, s); }
    Tensor& operator+=(double s) { return scalar_assign(RT_S_ADD, s); }
    Tensor& operator-=(double s) { return scalar_assign(RT_S_SUB, s); }
    Tensor& operator*=(double s) { return scalar_assign(RT_S_MUL, s); }
    Tensor& operator/=(double s) { return scalar_assign(RT_S_DIV, s); }
    Tensor& leaky_relu_inplace(double slope) { return scalar_assign(RT_S_LEAKY_RELU, slope); }
    Tensor& elu_inplace(double alpha) { return scalar_assign(RT_S_ELU, alpha); }
    Tensor& log_inplace(double base) { return scalar_assign(RT_S_LOG, base); }
    Tensor& log1p_inplace(double base) { return scalar_assign(RT_S_LOG1P, base); }

    // ---- unary ops: `t.f()` = owned() + `t.f_inplace()` in the reference (ops/unary/mod.rs:114-126), here one out-of-place pass
    // when the operand is a forward contiguous run ----------------------------------------------------------------------------------------
    Tensor& unary_inplace(int op) { backend_->apply_unary(op, *buf_, meta_); return *this; }
    Tensor unary(int op) const {
        if (one_pass_ok()) {
            Tensor r = like_row_major();
            backend_->apply_unary_to(op, *buf_, meta_.offset, size(), *r.buf_);
            return r;
        }
        Tensor r = owned();
        r.unary_inplace(op);
        return r;
    }
    Tensor operator-() const { return unary(RT_U_NEG); }
#define RT_TENSOR_UNARY(name, CODE)                            \
    Tensor name() const { return unary(CODE); }                \
    Tensor& name##_inplace() { return unary_inplace(CODE); }
    RT_TENSOR_UNARY(neg, RT_U_NEG) RT_TENSOR_UNARY(relu, RT_U_RELU) RT_TENSOR_UNARY(sigmoid, RT_U_SIGMOID) RT_TENSOR_UNARY(silu, RT_U_SILU)
    RT_TENSOR_UNARY(tanh, RT_U_TANH) RT_TENSOR_UNARY(abs, RT_U_ABS) RT_TENSOR_UNARY(sqrt, RT_U_SQRT) RT_TENSOR_UNARY(ln, RT_U_LN)
    RT_TENSOR_UNARY(expm1, RT_U_EXPM1) RT_TENSOR_UNARY(ln1p, RT_U_LN1P) RT_TENSOR_UNARY(floor, RT_U_FLOOR) RT_TENSOR_UNARY(ceil, RT_U_CEIL)
    RT_TENSOR_UNARY(round, RT_U_ROUND) RT_TENSOR_UNARY(trunc, RT_U_TRUNC) RT_TENSOR_UNARY(sin, RT_U_SIN) RT_TENSOR_UNARY(cos, RT_U_COS)
    RT_TENSOR_UNARY(tan, RT_U_TAN) RT_TENSOR_UNARY(asin, RT_U_ASIN) RT_TENSOR_UNARY(acos, RT_U_ACOS) RT_TENSOR_UNARY(atan, RT_U_ATAN)
    RT_TENSOR_UNARY(sinh, RT_U_SINH) RT_TENSOR_UNARY(cosh, RT_U_COSH) RT_TENSOR_UNARY(asinh, RT_U_ASINH) RT_TENSOR_UNARY(acosh, RT_U_ACOSH)
    RT_TENSOR_UNARY(atanh, RT_U_ATANH) RT_TENSOR_UNARY(rsqrt, RT_U_RSQRT) RT_TENSOR_UNARY(reciprocal, RT_U_RECIPROCAL)
    RT_TENSOR_UNARY(square, RT_U_SQUARE) RT_TENSOR_UNARY(cube, RT_U_CUBE) RT_TENSOR_UNARY(exp, RT_U_EXP) RT_TENSOR_UNARY(sign, RT_U_SIGN)
#undef RT_TENSOR_UNARY

    // ---- matmul / dot / outer (ops/linalg/matmul.rs:5-180) ------------------------------------------------------------------------------
    // (..., M, K) @ (..., K, N) -> (..., M, N); batch dims must match exactly.  An operand whose last two dims have no unit
    // stride, or whose batch dims do not collapse into one stride, is made row-major first (matmul.rs:42-62); so is one with
    // a negative stride, which the reference would cast to usize.
    Tensor matmul(const Tensor& rhs) const {
        if (rank() < 2) throw TensorError(ErrorKind::InvalidShape, "LHS tensor must have rank >= 2 for matmul");
        if (rhs.rank() < 2) throw TensorError(ErrorKind::InvalidShape, "RHS tensor must have rank >= 2 for matmul");
        auto prepared = [](const Tensor& t) {
            bool negative = false;
            for (int64_t s : t.meta_.strides) negative = negative || s < 0;
            return (negative || contiguity_type(t.meta_) == ContiguityTypes::None) ? t.gathered() : t;
        };
        const Tensor l = prepared(*this), r = prepared(rhs);
        const size_t lr = l.rank(), rr = r.rank();
        if (lr != rr) throw TensorError(ErrorKind::InvalidShape, "Both tensors must have the same rank >= 2");
        Shape batch(l.meta_.shape.begin(), l.meta_.shape.end() - 2);
        if (batch != Shape(r.meta_.shape.begin(), r.meta_.shape.end() - 2))
            throw TensorError(ErrorKind::SizeMismatch, "Batch dimensions must match for matmul");
        uint64_t b = 1;
        for (uint64_t d : batch) b *= d;
        const uint64_t m = l.meta_.shape[lr - 2], k = l.meta_.shape[lr - 1], kr = r.meta_.shape[rr - 2], n = r.meta_.shape[rr - 1];
        if (k != kr) throw TensorError(ErrorKind::SizeMismatch, "Inner matrix dimensions must match for matmul");
        Shape out_shape = batch;
        out_shape.push_back(m);
        out_shape.push_back(n);
        MetaTensor om = MetaTensor::row_major(out_shape);
        Tensor out(*backend_, backend_->alloc_uninit(dtype(), om.size()), om);
        backend_->matmul(*l.buf_, l.meta_, contiguity_type(l.meta_), *r.buf_, r.meta_, contiguity_type(r.meta_), *out.buf_, b, m, k, n);
        return out;
    }
    Tensor dot(const Tensor& rhs) const {
        if (rank() != 1 || rhs.rank() != 1) throw TensorError(ErrorKind::InvalidShape, "Dot product is only defined for 1-D tensors");
        return unsqueeze_at(0).matmul(rhs.unsqueeze_at(1)).squeeze();
    }
    Tensor outer(const Tensor& rhs) const {
        if (rank() != 1 || rhs.rank() != 1) throw TensorError(ErrorKind::InvalidShape, "Outer product is only defined for 1-D tensors");
        return unsqueeze_at(1).matmul(rhs.unsqueeze_at(0));
    }

    // ---- reductions ----------------------------------------------------------------------------------------------------------------------
    // Non-contiguous inputs are copied first (ops/reduction/mod.rs:346-408).  "Contiguous" here means a forward
    // row-major run: a reversed view is |stride|-contiguous for the reference and would reach its kernels with the
    // offset of the last element; it is gathered instead.
    Tensor reduce(ReductionOpTypes op, std::optional<size_t> axis) const {
        if (op == ReductionOpTypes::ArgMax || op == ReductionOpTypes::ArgMin) return arg_reduce(op, axis);
        if (!meta_.is_forward_contiguous()) return gathered().reduce(op, axis);
        if (!axis) {                                                           // Idx::Item (ops/reduction/mod.rs:272-285)
            Tensor out(*backend_, backend_->alloc_uninit(dtype(), 1), MetaTensor({}, {}, 0));
            backend_->apply_reduce_contiguous_flat(*buf_, *out.buf_, meta_.offset, meta_.size(), op);
            return out;
        }
        if (*axis >= rank()) throw TensorError(ErrorKind::InvalidDim, "reduction axis out of range");
        MetaTensor om = reduction_output_meta(meta_, axis);
        Tensor out(*backend_, backend_->alloc_uninit(dtype(), om.size()), om);
        backend_->apply_reduce(*buf_, meta_, *out.buf_, *axis, op);
        return out;
    }
    Tensor sum_at(size_t a) const { return reduce(ReductionOpTypes::Sum, a); }
    Tensor prod_at(size_t a) const { return reduce(ReductionOpTypes::Prod, a); }
    Tensor max_at(size_t a) const { return reduce(ReductionOpTypes::Max, a); }
    Tensor min_at(size_t a) const { return reduce(ReductionOpTypes::Min, a); }
    Tensor mean_at(size_t a) const { return reduce(ReductionOpTypes::Mean, a); }
    Tensor sum() const { return reduce(ReductionOpTypes::Sum, std::nullopt); }
    Tensor prod() const { return reduce(ReductionOpTypes::Prod, std::nullopt); }
    Tensor max() const { return reduce(ReductionOpTypes::Max, std::nullopt); }
    Tensor min() const { return reduce(ReductionOpTypes::Min, std::nullopt); }
    Tensor mean() const { return reduce(ReductionOpTypes::Mean, std::nullopt); }
    // the kinds only the reference's Cuda backend implements (ops/reduction/mod.rs:411-500)
    Tensor var_at(size_t a) const { return reduce(ReductionOpTypes::Variance, a); }
    Tensor pop_var_at(size_t a) const { return reduce(ReductionOpTypes::PopVariance, a); }
    Tensor std_at(size_t a, bool unbiased) const { return reduce(unbiased ? ReductionOpTypes::Stdev : ReductionOpTypes::PopStdev, a); }
    Tensor norm_at(size_t a, NormType n) const { return reduce(n == NormType::L1 ? ReductionOpTypes::NormL1 : ReductionOpTypes::NormL2, a); }
    Tensor l1_norm_at(size_t a) const { return norm_at(a, NormType::L1); }
    Tensor l2_norm_at(size_t a) const { return norm_at(a, NormType::L2); }
    Tensor logsumexp_at(size_t a) const { return reduce(ReductionOpTypes::LogSumExp, a); }
    Tensor argmax_at(size_t a) const { return arg_reduce(ReductionOpTypes::ArgMax, a); }
    Tensor argmin_at(size_t a) const { return arg_reduce(ReductionOpTypes::ArgMin, a); }
    Tensor var() const { return reduce(ReductionOpTypes::Variance, std::nullopt); }
    Tensor pop_var() const { return reduce(ReductionOpTypes::PopVariance, std::nullopt); }
    Tensor std(bool unbiased) const { return reduce(unbiased ? ReductionOpTypes::Stdev : ReductionOpTypes::PopStdev, std::nullopt); }
    Tensor norm(NormType n) const { return reduce(n == NormType::L1 ? ReductionOpTypes::NormL1 : ReductionOpTypes::NormL2, std::nullopt); }
    Tensor l1_norm() const { return norm(NormType::L1); }
    Tensor l2_norm() const { return norm(NormType::L2); }
    Tensor logsumexp() const { return reduce(ReductionOpTypes::LogSumExp, std::nullopt); }
    Tensor argmax() const { return arg_reduce(ReductionOpTypes::ArgMax, std::nullopt); }
    Tensor argmin() const { return arg_reduce(ReductionOpTypes::ArgMin, std::nullopt); }
    // do_argmax (ops/reduction/mod.rs:305-342): a u64 tensor of positions, rank-0 for the total form
    Tensor arg_reduce(ReductionOpTypes op, std::optional<size_t> axis) const {
        if (op != ReductionOpTypes::ArgMax && op != ReductionOpTypes::ArgMin)
            throw TensorError(ErrorKind::UnsupportedOperation, "arg_reduce takes ArgMax or ArgMin");
        if (!meta_.is_forward_contiguous()) return gathered().arg_reduce(op, axis);
        if (!axis) {
            Tensor out(*backend_, backend_->alloc_uninit(RT_U64, 1), MetaTensor({}, {}, 0));
            backend_->apply_argmax_contiguous_flat(*buf_, *out.buf_, meta_.offset, meta_.size(), op);
            return out;
        }
        if (*axis >= rank()) throw TensorError(ErrorKind::InvalidDim, "reduction axis out of range");
        MetaTensor om = reduction_output_meta(meta_, axis);
        Tensor out(*backend_, backend_->alloc_uninit(RT_U64, om.size()), om);
        backend_->apply_argmax(*buf_, meta_, *out.buf_, *axis, op);
        return out;
    }

    // PartialEq of tensors: same shape and the same addressed values
    bool equals(const Tensor& o) const {
        if (meta_.shape != o.meta_.shape || dtype() != o.dtype()) return false;
        Tensor a = gathered(), b = o.gathered();
        return backend_->equal(*a.buf_, *b.buf_);
    }

    // AsView::view_as (core/tensor.rs:120-122, 328-355): another shape over the same contiguous elements, no copy
    Tensor view_as(const Shape& shape) const { return with_meta(compute_view_as_parameters(meta_, shape)); }
    // AsTensor::reshape (core/tensor.rs:238-243): contiguous() and then the view_as meta on the new owner
    Tensor reshape(const Shape& shape) const {
        Tensor c = contiguous();
        c.meta_ = compute_view_as_parameters(c.meta_, shape);
        return c;
    }
    // metadata rewrite used by the autograd step (grad/backwards.rs:516-538 mutates `grad.meta` in place)
    void set_meta(const MetaTensor& m) { meta_ = m; }

  private:
    Tensor with_meta(const MetaTensor& m) const {
        Tensor t = *this;
        t.meta_ = m;
        t.is_view_ = true;
        return t;
    }
    Tensor gathered() const {
        Buf out = backend_->alloc_uninit(dtype(), meta_.size());
        backend_->gather(*buf_, meta_, *out);
        return Tensor(*backend_, out, MetaTensor::row_major(meta_.shape));
    }

    std::shared_ptr<Hip> backend_;
    Buf buf_;
    MetaTensor meta_;
    bool is_view_ = false;
};

// Typed face: TensorBase<T, Hip>.
template <class T>
class TensorBase : public Tensor {
  public:
    TensorBase() = default;
    TensorBase(const Tensor& t) : Tensor(t) {
        if (t.dtype() != dtype_of<T>::value) throw TensorError(ErrorKind::UnsupportedOperation, "dtype mismatch");
    }
    static TensorBase from_buf(const Hip& b, const std::vector<T>& v, const Shape& shape) {
        return TensorBase(Tensor::from_buf(b, dtype_of<T>::value, v.data(), v.size(), shape));
    }
    static TensorBase zeros(const Hip& b, const Shape& s) { return TensorBase(Tensor::zeros(b, dtype_of<T>::value, s)); }
    static TensorBase ones(const Hip& b, const Shape& s) { return TensorBase(Tensor::ones(b, dtype_of<T>::value, s)); }
    static TensorBase max(const Hip& b, const Shape& s) { return TensorBase(Tensor::max(b, dtype_of<T>::value, s)); }
    static TensorBase min(const Hip& b, const Shape& s) { return TensorBase(Tensor::min(b, dtype_of<T>::value, s)); }
    static TensorBase scalar(const Hip& b, T v) { return TensorBase(Tensor::scalar(b, Scalar::of<T>(v))); }
    static TensorBase column(const Hip& b, const std::vector<T>& v) { return TensorBase(Tensor::column(b, dtype_of<T>::value, v.data(), v.size())); }
    static TensorBase row(const Hip& b, const std::vector<T>& v) { return TensorBase(Tensor::row(b, dtype_of<T>::value, v.data(), v.size())); }
    template <class N> TensorBase<N> into_dtype() const { return TensorBase<N>(Tensor::into_dtype(dtype_of<N>::value)); }
    std::vector<T> to_vec() const {
        std::vector<T> out(size());
        to_host(out.data());
        return out;
    }
    T at(const std::vector<uint64_t>& idx) const { return get(idx).template as<T>(); }
    T item_value() const { return item().template as<T>(); }
};

}  // namespace rt

// `rt::Hip`: the host-side counterpart of `impl Backend for ...` (libs/rtensors/src/backend/mod.rs:216-485) over the C
// ABI of librt_hip.so.  Method names and argument meaning follow the trait; `Buf` is `HipBuf` (device pointer + length +
// dtype, what `CudaBuf` is in backend/cuda.rs:53-57).  The only dependency is include/rt_hip.h: no HIP headers, so this
// layer builds with a plain host compiler, the way a Rust FFI binding would.
#pragma once

#include <cmath>
#include <limits>
#include <cstring>
#include <memory>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/rt_hip.h"
#include "rt_meta.hpp"

namespace rt {

// ---- dtypes (core/value.rs:567-581) -----------------------------------------------------------------------------------
struct boolean { uint8_t v; bool operator==(const boolean& o) const { return v == o.v; } };
typedef unsigned __int128 u128;
typedef __int128 i128;

template <class T> struct dtype_of;
#define RT_DT(T, CODE) template <> struct dtype_of<T> { static constexpr int value = CODE; }
RT_DT(uint8_t, RT_U8); RT_DT(int8_t, RT_I8); RT_DT(uint16_t, RT_U16); RT_DT(int16_t, RT_I16); RT_DT(uint32_t, RT_U32); RT_DT(u128, RT_U128);
RT_DT(int32_t, RT_I32); RT_DT(uint64_t, RT_U64); RT_DT(int64_t, RT_I64); RT_DT(i128, RT_I128); RT_DT(float, RT_F32); RT_DT(double, RT_F64);
RT_DT(boolean, RT_BOOL);
#undef RT_DT

// One element of any dtype, carried by value across the C ABI.
struct Scalar {
    int dtype = RT_F32;
    alignas(16) unsigned char bytes[16] = {0};
    template <class T> static Scalar of(T v) { Scalar s; s.dtype = dtype_of<T>::value; std::memcpy(s.bytes, &v, sizeof(T)); return s; }
    template <class T> T as() const { T v; std::memcpy(&v, bytes, sizeof(T)); return v; }
    // double -> integer with the meaning of Rust's `as` (core/value.rs:268-312 uses it for every conversion): NaN is 0, values
    // beyond the type's range saturate, the rest truncate toward zero.  A plain C++ cast is undefined for the first two.
    template <class T> static T int_from_double(double x) {
        if (x != x) return (T)0;
        constexpr bool is_signed = (T)-1 < (T)0;
        constexpr int bits = (int)(8 * sizeof(T)) - (is_signed ? 1 : 0);
        const double hi = std::ldexp(1.0, bits);                        // first value above the range, exact in double
        // through u128 so that no signed shift overflows: the conversion back to T is modular
        const T max_v = is_signed ? (T)(((u128)1 << (bits & 127)) - 1) : (T)~(T)0;
        const T min_v = is_signed ? (T)((u128)1 << (bits & 127)) : (T)0;
        if (x >= hi) return max_v;
        if (is_signed ? x < -hi : x <= -1.0) return min_v;
        if (!is_signed && x < 0.0) return (T)0;                         // (-1, 0) truncates to 0
        return (T)x;
    }
    // numeric literal -> element of `dtype` (what `T::from` does for the scalar operand of `tensor + 3`)
    static Scalar from_double(int dtype, double x) {
        switch (dtype) {
            case RT_U8: return of<uint8_t>(int_from_double<uint8_t>(x));    case RT_I8: return of<int8_t>(int_from_double<int8_t>(x));
            case RT_U16: return of<uint16_t>(int_from_double<uint16_t>(x)); case RT_I16: return of<int16_t>(int_from_double<int16_t>(x));
            case RT_U32: return of<uint32_t>(int_from_double<uint32_t>(x)); case RT_I32: return of<int32_t>(int_from_double<int32_t>(x));
            case RT_U64: return of<uint64_t>(int_from_double<uint64_t>(x)); case RT_I64: return of<int64_t>(int_from_double<int64_t>(x));
            case RT_U128: return of<u128>(int_from_double<u128>(x));        case RT_I128: return of<i128>(int_from_double<i128>(x));
            case RT_F32: return of<float>((float)x); case RT_F64: return of<double>(x);
            case RT_BOOL: return of<boolean>(boolean{(uint8_t)(x != 0)});
        }
        throw TensorError(ErrorKind::UnsupportedOperation, "unknown dtype code");
    }
    // T::MIN / T::MAX of the element type (core/value.rs:496-508, 703-704): the lowest / highest finite value for floats
    static Scalar limit(int dtype, bool highest) {
        switch (dtype) {
            case RT_U8: return of<uint8_t>(highest ? UINT8_MAX : 0); case RT_I8: return of<int8_t>(highest ? INT8_MAX : INT8_MIN);
            case RT_U16: return of<uint16_t>(highest ? UINT16_MAX : 0); case RT_I16: return of<int16_t>(highest ? INT16_MAX : INT16_MIN);
            case RT_U32: return of<uint32_t>(highest ? UINT32_MAX : 0); case RT_I32: return of<int32_t>(highest ? INT32_MAX : INT32_MIN);
            case RT_U64: return of<uint64_t>(highest ? UINT64_MAX : 0); case RT_I64: return of<int64_t>(highest ? INT64_MAX : INT64_MIN);
            case RT_U128: return of<u128>(highest ? ~(u128)0 : (u128)0);
            case RT_I128: return of<i128>(highest ? (i128)(~(u128)0 >> 1) : -(i128)(~(u128)0 >> 1) - 1);
            case RT_F32: return of<float>(highest ? std::numeric_limits<float>::max() : std::numeric_limits<float>::lowest());
            case RT_F64: return of<double>(highest ? std::numeric_limits<double>::max() : std::numeric_limits<double>::lowest());
            case RT_BOOL: return of<boolean>(boolean{(uint8_t)(highest ? 1 : 0)});
        }
        throw TensorError(ErrorKind::UnsupportedOperation, "unknown dtype code");
    }
    double to_double() const {
        switch (dtype) {
            case RT_U8: return as<uint8_t>(); case RT_I8: return as<int8_t>(); case RT_U16: return as<uint16_t>(); case RT_I16: return as<int16_t>();
            case RT_U32: return as<uint32_t>(); case RT_I32: return as<int32_t>(); case RT_U64: return (double)as<uint64_t>();
            case RT_I64: return (double)as<int64_t>(); case RT_U128: return (double)as<u128>(); case RT_I128: return (double)as<i128>();
            case RT_F32: return as<float>(); case RT_F64: return as<double>(); case RT_BOOL: return as<boolean>().v;
        }
        return 0;
    }
};

inline ErrorKind kind_of_status(int32_t st) {
    switch (st) {
        case RT_E_DTYPE: case RT_E_RANK: return ErrorKind::UnsupportedOperation;
        case RT_E_OUT_OF_BOUNDS: return ErrorKind::IdxOutOfBounds;
        case RT_E_WRONG_DIMS: return ErrorKind::WrongDims;
        case RT_E_SIZE_MISMATCH: return ErrorKind::SizeMismatch;
        case RT_E_ARITH: return ErrorKind::Panic;
        case RT_E_INVALID: return ErrorKind::InvalidShape;
        default: return ErrorKind::HipError;
    }
}
inline void check(int32_t st) {
    if (st != RT_OK) throw TensorError(kind_of_status(st), rt_last_error());
}

// ops/base.rs:7-12, ops/reduction/mod.rs:141-175
enum class BinaryOpType : int { Add = RT_ADD, Sub = RT_SUB, Mul = RT_MUL, Div = RT_DIV };
// ReductionOpTypes (ops/reduction/mod.rs:141-175).  The variants that carry a payload there -- Variance { unbiased },
// Stdev { unbiased }, Norm(L1 | L2) -- are spelled out, with the payload in the flag bits the C ABI takes.
enum class ReductionOpTypes : int {
    Sum = RT_R_SUM, Prod = RT_R_PROD, Max = RT_R_MAX, Min = RT_R_MIN, Mean = RT_R_MEAN,
    PopVariance = RT_R_VARIANCE, Variance = RT_R_VARIANCE | RT_R_FLAG_UNBIASED,
    PopStdev = RT_R_VARIANCE | RT_R_FLAG_STD, Stdev = RT_R_VARIANCE | RT_R_FLAG_STD | RT_R_FLAG_UNBIASED,
    LogSumExp = RT_R_LOGSUMEXP, NormL1 = RT_R_NORM | RT_R_FLAG_L1, NormL2 = RT_R_NORM | RT_R_FLAG_L2,
    ArgMax = RT_R_ARGMAX, ArgMin = RT_R_ARGMIN
};
enum class NormType { L1, L2 };                                   // ops/reduction/mod.rs:203-206

class Hip;

// Owns device memory; dropping it returns the block to the context's caching allocator.
class HipBuf {
  public:
    HipBuf(std::shared_ptr<rt_ctx> ctx, void* ptr, uint64_t len, int dtype) : ctx_(std::move(ctx)), ptr_(ptr), len_(len), dtype_(dtype) {}
    HipBuf(const HipBuf&) = delete;
    HipBuf& operator=(const HipBuf&) = delete;
    ~HipBuf() { if (ptr_) rt_free(ctx_.get(), ptr_); }
    void* ptr() const { return ptr_; }
    uint64_t len() const { return len_; }
    int dtype() const { return dtype_; }
  private:
    std::shared_ptr<rt_ctx> ctx_;
    void* ptr_;
    uint64_t len_;
    int dtype_;
};
using Buf = std::shared_ptr<HipBuf>;

// `Hip: Clone` shares one context (device + stream + allocator), like the Arc'd CUDA context of backend/cuda.rs:38-51.
class Hip {
  public:
    explicit Hip(int device = 0) {
        rt_ctx* c = nullptr;
        check(rt_ctx_create(device, &c));
        ctx_ = std::shared_ptr<rt_ctx>(c, [](rt_ctx* p) { rt_ctx_destroy(p); });
    }
    static Hip create(int device = 0) { return Hip(device); }       // Backend::new
    rt_ctx* raw() const { return ctx_.get(); }
    void sync() const { check(rt_sync(raw())); }

    // ---- buffers (backend/mod.rs:225-235) --------------------------------------------------------------------------
    Buf alloc(int dtype, uint64_t len) const {
        void* p = nullptr;
        check(rt_alloc(raw(), dtype, len, &p));
        return std::make_shared<HipBuf>(ctx_, p, len, dtype);
    }
    Buf alloc_uninit(int dtype, uint64_t len) const {
        void* p = nullptr;
        check(rt_alloc_uninit(raw(), dtype, len, &p));
        return std::make_shared<HipBuf>(ctx_, p, len, dtype);
    }
    Buf alloc_from_slice(int dtype, const void* src, uint64_t len) const {
        void* p = nullptr;
        check(rt_alloc_from_slice(raw(), dtype, src, len, &p));
        return std::make_shared<HipBuf>(ctx_, p, len, dtype);
    }
    void copy_from_slice(HipBuf& dst, const void* src, uint64_t len) const { check(rt_copy_from_slice(raw(), dst.dtype(), dst.ptr(), dst.len(), src, len)); }
    void copy_range_within(HipBuf& dst, const HipBuf& src, uint64_t dst_offset, uint64_t src_offset, uint64_t len) const {
        check(rt_copy_range_within(raw(), dst.dtype(), dst.ptr(), dst.len(), src.ptr(), src.len(), dst_offset, src_offset, len));
    }
    Scalar read(const HipBuf& buf, uint64_t offset) const {
        Scalar s;
        s.dtype = buf.dtype();
        check(rt_read(raw(), buf.dtype(), buf.ptr(), buf.len(), offset, s.bytes));
        return s;
    }
    void write(HipBuf& buf, uint64_t offset, const Scalar& v) const { check(rt_write(raw(), buf.dtype(), buf.ptr(), buf.len(), offset, v.bytes)); }
    uint64_t len(const HipBuf& buf) const { return buf.len(); }
    Buf copy(const HipBuf& src) const {
        void* p = nullptr;
        check(rt_copy(raw(), src.dtype(), src.ptr(), src.len(), &p));
        return std::make_shared<HipBuf>(ctx_, p, src.len(), src.dtype());
    }
    void dump(const HipBuf& src, void* host_dst) const { check(rt_dump(raw(), src.dtype(), src.ptr(), src.len(), host_dst)); }
    void convert(const HipBuf& src, HipBuf& dst) const { check(rt_convert(raw(), src.dtype(), src.ptr(), src.len(), dst.dtype(), dst.ptr(), dst.len())); }
    bool equal(const HipBuf& a, const HipBuf& b) const {
        if (a.dtype() != b.dtype()) return false;
        int32_t eq = 0;
        check(rt_equal(raw(), a.dtype(), a.ptr(), a.len(), b.ptr(), b.len(), &eq));
        return eq != 0;
    }

    // ---- fill / unary / scalar.  The trait's default methods pick contiguous / 1-D strided / N-d from |stride|
    // contiguity (backend/mod.rs:15-213); here the whole view goes down and the C side canonicalises it with signed
    // strides, so a reversed view is walked backwards instead of being mistaken for a forward run. ------------------
    void fill(HipBuf& buf, const Scalar& v, const MetaTensor& m) const {
        check(rt_fill_nd(raw(), buf.dtype(), buf.ptr(), buf.len(), v.bytes, m.offset, (int32_t)m.rank(), m.shape.data(), m.strides.data()));
    }
    void fill_contiguous(HipBuf& buf, const Scalar& v, uint64_t start, uint64_t len) const {
        check(rt_fill_contiguous(raw(), buf.dtype(), buf.ptr(), buf.len(), v.bytes, start, len));
    }
    void fill_1d_strided(HipBuf& buf, const Scalar& v, uint64_t offset, int64_t stride, uint64_t len) const {
        check(rt_fill_1d_strided(raw(), buf.dtype(), buf.ptr(), buf.len(), v.bytes, offset, stride, len));
    }
    void apply_unary(int op, HipBuf& buf, const MetaTensor& m) const {
        check(rt_unary_nd(raw(), buf.dtype(), op, buf.ptr(), buf.len(), m.offset, (int32_t)m.rank(), m.shape.data(), m.strides.data()));
    }
    void apply_unary_contiguous(int op, HipBuf& buf, uint64_t start, uint64_t len) const {
        check(rt_unary_contiguous(raw(), buf.dtype(), op, buf.ptr(), buf.len(), start, len));
    }
    void apply_unary_1d_strided(int op, HipBuf& buf, uint64_t offset, int64_t stride, uint64_t len) const {
        check(rt_unary_1d_strided(raw(), buf.dtype(), op, buf.ptr(), buf.len(), offset, stride, len));
    }
    void scalar_apply(int op, HipBuf& buf, const Scalar& v, const MetaTensor& m) const {
        check(rt_scalar_nd(raw(), buf.dtype(), op, buf.ptr(), buf.len(), v.bytes, m.offset, (int32_t)m.rank(), m.shape.data(), m.strides.data()));
    }
    // out-of-place forms over a contiguous run: dst[0 .. len) = op(src[start .. start + len)) in one pass
    void apply_unary_to(int op, const HipBuf& src, uint64_t start, uint64_t len, HipBuf& dst) const {
        check(rt_unary_to(raw(), src.dtype(), op, src.ptr(), src.len(), start, len, dst.ptr(), dst.len()));
    }
    void scalar_apply_to(int op, const HipBuf& src, const Scalar& v, uint64_t start, uint64_t len, HipBuf& dst) const {
        check(rt_scalar_to(raw(), src.dtype(), op, src.ptr(), src.len(), v.bytes, start, len, dst.ptr(), dst.len()));
    }
    // the trait's named methods (apply_relu, scalar_apply_add, ...) in terms of the op codes
#define RT_UNARY_METHOD(name, CODE) void apply_##name(HipBuf& buf, const MetaTensor& m) const { apply_unary(CODE, buf, m); }
    RT_UNARY_METHOD(neg, RT_U_NEG) RT_UNARY_METHOD(relu, RT_U_RELU) RT_UNARY_METHOD(sigmoid, RT_U_SIGMOID) RT_UNARY_METHOD(silu, RT_U_SILU)
    RT_UNARY_METHOD(tanh, RT_U_TANH) RT_UNARY_METHOD(abs, RT_U_ABS) RT_UNARY_METHOD(sqrt, RT_U_SQRT) RT_UNARY_METHOD(ln, RT_U_LN)
    RT_UNARY_METHOD(expm1, RT_U_EXPM1) RT_UNARY_METHOD(ln1p, RT_U_LN1P) RT_UNARY_METHOD(floor, RT_U_FLOOR) RT_UNARY_METHOD(ceil, RT_U_CEIL)
    RT_UNARY_METHOD(round, RT_U_ROUND) RT_UNARY_METHOD(trunc, RT_U_TRUNC) RT_UNARY_METHOD(sin, RT_U_SIN) RT_UNARY_METHOD(cos, RT_U_COS)
    RT_UNARY_METHOD(tan, RT_U_TAN) RT_UNARY_METHOD(asin, RT_U_ASIN) RT_UNARY_METHOD(acos, RT_U_ACOS) RT_UNARY_METHOD(atan, RT_U_ATAN)
    RT_UNARY_METHOD(sinh, RT_U_SINH) RT_UNARY_METHOD(cosh, RT_U_COSH) RT_UNARY_METHOD(asinh, RT_U_ASINH) RT_UNARY_METHOD(acosh, RT_U_ACOSH)
    RT_UNARY_METHOD(atanh, RT_U_ATANH) RT_UNARY_METHOD(rsqrt, RT_U_RSQRT) RT_UNARY_METHOD(reciprocal, RT_U_RECIPROCAL)
    RT_UNARY_METHOD(square, RT_U_SQUARE) RT_UNARY_METHOD(cube, RT_U_CUBE) RT_UNARY_METHOD(exp, RT_U_EXP) RT_UNARY_METHOD(sign, RT_U_SIGN)
#undef RT_UNARY_METHOD
#define RT_SCALAR_METHOD(name, CODE) void scalar_apply_##name(HipBuf& buf, const Scalar& v, const MetaTensor& m) const { scalar_apply(CODE, buf, v, m); }
    RT_SCALAR_METHOD(add, RT_S_ADD) RT_SCALAR_METHOD(sub, RT_S_SUB) RT_SCALAR_METHOD(mul, RT_S_MUL) RT_SCALAR_METHOD(div, RT_S_DIV)
    RT_SCALAR_METHOD(log, RT_S_LOG) RT_SCALAR_METHOD(log1p, RT_S_LOG1P) RT_SCALAR_METHOD(leaky_relu, RT_S_LEAKY_RELU) RT_SCALAR_METHOD(elu, RT_S_ELU)
#undef RT_SCALAR_METHOD

    // ---- broadcast (backend/mod.rs:296-309): operands pre-broadcast to one shape; dst may be left ---------------------
    void broadcast(const HipBuf& left, const MetaTensor& lm, const HipBuf& right, const MetaTensor& rm, HipBuf& dst, const MetaTensor& dm,
                   BinaryOpType op) const {
        if (lm.shape != dm.shape || rm.shape != dm.shape)
            throw TensorError(ErrorKind::InvalidShape, "broadcast operands must be pre-broadcast to the output shape");
        check(rt_broadcast(raw(), dst.dtype(), (int)op, (int32_t)dm.rank(), dm.shape.data(), left.ptr(), left.len(), lm.offset, lm.strides.data(),
                           right.ptr(), right.len(), rm.offset, rm.strides.data(), dst.ptr(), dst.len(), dm.offset, dm.strides.data()));
    }

    // ---- reductions (backend/mod.rs:357-409) -------------------------------------------------------------------------
    void apply_reduce_contiguous_flat(const HipBuf& src, HipBuf& dst, uint64_t start, uint64_t len, ReductionOpTypes op) const {
        check(rt_reduce_flat(raw(), src.dtype(), (int)op, src.ptr(), src.len(), dst.ptr(), dst.len(), start, len));
    }
    void apply_reduce_contiguous_nd(const HipBuf& src, const MetaTensor& sm, HipBuf& dst, size_t dim, ReductionOpTypes op) const {
        check(rt_reduce_nd(raw(), src.dtype(), (int)op, src.ptr(), src.len(), sm.offset, (int32_t)sm.rank(), sm.shape.data(), sm.strides.data(),
                           dst.ptr(), dst.len(), (int32_t)dim));
    }
    // backend/mod.rs:375-409
    void apply_reduce(const HipBuf& src, const MetaTensor& sm, HipBuf& dst, size_t dim, ReductionOpTypes op) const {
        if (!sm.is_contiguous()) throw TensorError(ErrorKind::WrongDims, "Reduction over non-contiguous tensors is not implemented yet.");
        if (sm.rank() == 1) apply_reduce_contiguous_flat(src, dst, sm.offset, sm.size(), op);
        else apply_reduce_contiguous_nd(src, sm, dst, dim, op);
    }
    // Backend::apply_argmax_contiguous_flat / _nd / apply_argmax (backend/mod.rs:412-463): dst is a u64 buffer
    void apply_argmax_contiguous_flat(const HipBuf& src, HipBuf& dst, uint64_t start, uint64_t len, ReductionOpTypes op) const {
        if (dst.dtype() != RT_U64) throw TensorError(ErrorKind::UnsupportedOperation, "argmax writes u64 indices");
        check(rt_argmax_flat(raw(), src.dtype(), (int)op, src.ptr(), src.len(), (uint64_t*)dst.ptr(), dst.len(), start, len));
    }
    void apply_argmax_contiguous_nd(const HipBuf& src, const MetaTensor& sm, HipBuf& dst, size_t dim, ReductionOpTypes op) const {
        if (dst.dtype() != RT_U64) throw TensorError(ErrorKind::UnsupportedOperation, "argmax writes u64 indices");
        check(rt_argmax_nd(raw(), src.dtype(), (int)op, src.ptr(), src.len(), sm.offset, (int32_t)sm.rank(), sm.shape.data(), sm.strides.data(),
                           (uint64_t*)dst.ptr(), dst.len(), (int32_t)dim));
    }
    void apply_argmax(const HipBuf& src, const MetaTensor& sm, HipBuf& dst, size_t dim, ReductionOpTypes op) const {
        if (!sm.is_contiguous()) throw TensorError(ErrorKind::WrongDims, "Reduction over non-contiguous tensors is not implemented yet.");
        if (sm.rank() == 1) apply_argmax_contiguous_flat(src, dst, sm.offset, sm.size(), op);
        else apply_argmax_contiguous_nd(src, sm, dst, dim, op);
    }
    // conv2d sits behind the same trait but outside this path; it reports an error instead of the Cpu backend's todo!() panic
    // (backend/cpu.rs:473-481).
    void apply_conv_2d() const { throw TensorError(ErrorKind::UnsupportedOperation, "conv2d is not implemented by the Hip backend"); }

    // ---- BackendMatMul::matmul (backend/mod.rs:474-485) ---------------------------------------------------------------------
    void matmul(const HipBuf& lhs, const MetaTensor& lm, ContiguityTypes lc, const HipBuf& rhs, const MetaTensor& rm, ContiguityTypes rc, HipBuf& dst,
                uint64_t b, uint64_t m, uint64_t k, uint64_t n) const {
        check(rt_matmul(raw(), dst.dtype(), lhs.ptr(), lhs.len(), lm.offset, (int32_t)lm.rank(), lm.shape.data(), lm.strides.data(), (int32_t)lc,
                        rhs.ptr(), rhs.len(), rm.offset, (int32_t)rm.rank(), rm.shape.data(), rm.strides.data(), (int32_t)rc, dst.ptr(), dst.len(),
                        b, m, k, n));
    }

    // ---- fused passes of y = relu(x + bias), mean_l1_loss(y, t) and their backward (no counterpart in the trait; every element-wise
    // result is bit for bit what the separate calls give) -----------------------------------------------------------------------
    void fused_bias_relu(const HipBuf& x, const HipBuf& bias, HipBuf& y, uint64_t rows, uint64_t cols) const {
        check(rt_fused_bias_relu(raw(), y.dtype(), x.ptr(), x.len(), bias.ptr(), bias.len(), y.ptr(), y.len(), rows, cols));
    }
    void fused_l1_forward(const HipBuf& y, const HipBuf& target, HipBuf& gmap, HipBuf& loss, uint64_t n) const {
        check(rt_fused_l1_forward(raw(), y.dtype(), y.ptr(), y.len(), target.ptr(), target.len(), gmap.ptr(), gmap.len(), loss.ptr(), loss.len(), n));
    }
    void fused_l1_relu_backward(const HipBuf& gmap, const HipBuf& y, const HipBuf& upstream, HipBuf& dbias, uint64_t rows, uint64_t cols) const {
        check(rt_fused_l1_relu_backward(raw(), y.dtype(), gmap.ptr(), gmap.len(), y.ptr(), y.len(), upstream.ptr(), upstream.len(), dbias.ptr(), dbias.len(),
                                        rows, cols));
    }

    // the same step without a stored gradient map
    void fused_bias_relu_l1(const HipBuf& x, const HipBuf& bias, const HipBuf& target, HipBuf& y, HipBuf& loss, uint64_t rows, uint64_t cols) const {
        check(rt_fused_bias_relu_l1(raw(), y.dtype(), x.ptr(), x.len(), bias.ptr(), bias.len(), target.ptr(), target.len(), y.ptr(), y.len(), loss.ptr(),
                                    loss.len(), rows, cols));
    }
    void fused_l1_relu_backward_t(const HipBuf& y, const HipBuf& target, const HipBuf& upstream, HipBuf& dbias, uint64_t rows, uint64_t cols) const {
        check(rt_fused_l1_relu_backward_t(raw(), y.dtype(), y.ptr(), y.len(), target.ptr(), target.len(), upstream.ptr(), upstream.len(), dbias.ptr(),
                                          dbias.len(), rows, cols));
    }

    // row-major copy of a view (what TensorView::owned needs, core/tensor.rs:299-325) in one launch
    void gather(const HipBuf& src, const MetaTensor& m, HipBuf& dst) const {
        check(rt_gather(raw(), src.dtype(), src.ptr(), src.len(), m.offset, (int32_t)m.rank(), m.shape.data(), m.strides.data(), dst.ptr(), dst.len()));
    }

  private:
    std::shared_ptr<rt_ctx> ctx_;
};

}  // namespace rt

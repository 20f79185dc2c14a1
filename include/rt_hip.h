/*
 * rt_hip.h -- C ABI of the MI355X (gfx950) backend for rtensors.
 *
 * This is the boundary a Rust `impl Backend for Hip` binds (one entry point per required method family of
 * `trait Backend`, libs/rtensors/src/backend/mod.rs:216-472, in the de-genericised form the reference already
 * uses for its remote protocol, backend/remote/protocol.rs:246-291).  Plain pointers and sizes only.
 *
 * Conventions
 *   - Every function returns an rt_status (0 = ok).  Nothing aborts; a bad descriptor is an error code, never a
 *     device fault (checks follow backend/remote/server.rs:241-380).  rt_last_error() gives the message of the
 *     last failure on the calling thread.
 *   - `dtype` uses the reference's DType codes (core/value.rs:567-581), binary ops its BinaryOpType codes
 *     (ops/base.rs:7-12), reductions its ReductionOpTypes codes (ops/reduction/mod.rs:161-175), unary and scalar
 *     ops the declaration order of UnaryOp / ScalarOp (backend/remote/protocol.rs:213-232).
 *   - Buffers are device pointers returned by rt_alloc*; every call that touches a buffer also takes its length
 *     in elements so that extents can be validated.  Offsets, strides and lengths are in elements.
 *   - Work is enqueued on the context's stream and returns immediately; rt_read / rt_dump / rt_equal /
 *     rt_sync wait for it (as the reference's Cuda backend does, backend/cuda.rs:164-185, 719-836).
 *   - A context may be used from several host threads; calls are serialised internally.
 */
#ifndef RT_HIP_H
#define RT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct rt_ctx rt_ctx;

typedef enum rt_status {
    RT_OK = 0,
    RT_E_INVALID = 1,      /* malformed argument (null pointer, unknown code, shape/stride mismatch) */
    RT_E_DTYPE = 2,        /* dtype/op combination the trait bounds of the reference do not admit, or not built */
    RT_E_OUT_OF_BOUNDS = 3,/* a descriptor addresses elements outside its buffer (TensorError::IdxOutOfBounds) */
    RT_E_HIP = 4,          /* HIP runtime failure; see rt_last_error() */
    RT_E_OOM = 5,          /* device allocation failed */
    RT_E_RANK = 6,         /* more than RT_MAX_RANK dims remain after collapsing */
    RT_E_ARITH = 7,        /* integer division by zero or MIN / -1, mean over an empty integer axis (the reference panics) */
    RT_E_WRONG_DIMS = 8,   /* TensorError::WrongDims: reduction source is not contiguous (backend/mod.rs:386-390) */
    RT_E_SIZE_MISMATCH = 9 /* TensorError::SizeMismatch (backend/cpu.rs:151-161) */
} rt_status;

/* core/value.rs:567-581 */
typedef enum rt_dtype {
    RT_U8 = 0, RT_I8 = 1, RT_U16 = 2, RT_I16 = 3, RT_U32 = 4, RT_U128 = 5, RT_I32 = 6, RT_U64 = 7, RT_I64 = 8,
    RT_I128 = 9, RT_F32 = 10, RT_F64 = 11, RT_BOOL = 12
} rt_dtype;

/* ops/base.rs:7-12 */
typedef enum rt_binary_op { RT_ADD = 0, RT_SUB = 1, RT_MUL = 2, RT_DIV = 3 } rt_binary_op;

/* backend/remote/protocol.rs:226-232 */
typedef enum rt_scalar_op {
    RT_S_ADD = 0, RT_S_SUB = 1, RT_S_MUL = 2, RT_S_DIV = 3, RT_S_LOG = 4, RT_S_LOG1P = 5, RT_S_LEAKY_RELU = 6, RT_S_ELU = 7,
    /* No op of its own in the reference: x > 0 ? 1 : s, the leaky-ReLU gradient map its autograd builds one element at a
     * time with get/set (ops/scalar/mod.rs:149-166). */
    RT_S_LEAKY_GRAD = 8
} rt_scalar_op;

/* backend/remote/protocol.rs:213-224 */
typedef enum rt_unary_op {
    RT_U_NEG = 0, RT_U_RELU, RT_U_SIGMOID, RT_U_SILU, RT_U_TANH, RT_U_ABS, RT_U_SQRT, RT_U_LN, RT_U_EXPM1, RT_U_LN1P,
    RT_U_FLOOR, RT_U_CEIL, RT_U_ROUND, RT_U_TRUNC, RT_U_SIN, RT_U_COS, RT_U_TAN, RT_U_ASIN, RT_U_ACOS, RT_U_ATAN,
    RT_U_SINH, RT_U_COSH, RT_U_ASINH, RT_U_ACOSH, RT_U_ATANH, RT_U_RSQRT, RT_U_RECIPROCAL, RT_U_SQUARE, RT_U_CUBE,
    RT_U_EXP, RT_U_SIGN, RT_U_COUNT,
    /* Two maps with no op of their own in the reference: its autograd builds them one element at a time with get/set
     * (ops/unary/mod.rs:213-252), which on a device backend is one round trip per element. */
    RT_U_STEP = 31,      /* x > 0 ? 1 : 0   -- the ReLU gradient map (ops/unary/mod.rs:234-252) */
    RT_U_ABS_GRAD = 32,  /* x > 0 ? 1 : -1  -- the Abs gradient map  (ops/unary/mod.rs:213-232) */
    RT_U_EXT_COUNT = 33
} rt_unary_op;

/* ReductionOpTypes::get_code, ops/reduction/mod.rs:161-175.  The low byte is the reference's code; the variants that carry a
 * payload (Variance { unbiased }, Stdev { unbiased }, Norm(L1 | L2)) put it into the flag bits, the same three facts that
 * populate_reduction_settings (backend/cuda.rs:1750-1774) hands to the reference's kernels as `ReductionSettings`. */
#define RT_R_FLAG_UNBIASED 0x100 /* divide by n - 1 (var_at, std_at(.., true)); without it by n (pop_var_at) */
#define RT_R_FLAG_STD 0x200      /* square root of the variance */
#define RT_R_FLAG_L1 0x100       /* norm: sum |x| */
#define RT_R_FLAG_L2 0x200       /* norm: sqrt(sum x^2) */
typedef enum rt_reduce_op {
    RT_R_SUM = 1, RT_R_PROD = 2, RT_R_MAX = 3, RT_R_MIN = 4, RT_R_MEAN = 5,
    RT_R_VARIANCE = 6,           /* | RT_R_FLAG_UNBIASED | RT_R_FLAG_STD */
    RT_R_LOGSUMEXP = 7,
    RT_R_NORM = 8,               /* | RT_R_FLAG_L1 or RT_R_FLAG_L2 (one of them is required) */
    RT_R_ARGMAX = 9, RT_R_ARGMIN = 10 /* rt_argmax_flat / rt_argmax_nd only */
} rt_reduce_op;

#define RT_MAX_RANK 8        /* dims a kernel descriptor holds after size-1 removal and merging of adjacent dims */
#define RT_MAX_INPUT_RANK 128 /* the reference's own cap on rank (core/primitives.rs:377-383) */

/* ---- context ------------------------------------------------------------------------------------------------
 * Replaces the lazily built per-device singleton + default stream of backend/cuda.rs:38-51, 143-185.
 * device >= 0 names the device; device == -1 takes the environment variable RT_HIP_DEVICE (a device index; 0 when it is unset).
 * A malformed or out-of-range value is RT_E_INVALID. */
int32_t rt_ctx_create(int32_t device, rt_ctx** out);
int32_t rt_ctx_destroy(rt_ctx* ctx);
int32_t rt_sync(rt_ctx* ctx);                       /* Cuda::sync, backend/cuda.rs:164-185 */
const char* rt_last_error(void);                    /* message of the last failing call on this thread */
const char* rt_status_name(int32_t status);
int32_t rt_dtype_size(int32_t dtype);               /* bytes per element, 0 for an unknown code */
int32_t rt_device_count(int32_t* out);

/* ---- buffers and transfers (Backend::alloc .. dump, backend/mod.rs:225-233; Cpu backend/cpu.rs:147-243) ------- */
/* Backend::alloc: `len` elements, zero-initialised like the Cpu backend's vec![T::default(); len]. */
int32_t rt_alloc(rt_ctx* ctx, int32_t dtype, uint64_t len, void** out);
/* Same without the zero fill, for outputs every element of which is about to be written. */
int32_t rt_alloc_uninit(rt_ctx* ctx, int32_t dtype, uint64_t len, void** out);
/* Backend::alloc_from_slice: allocate and upload `len` host elements. */
int32_t rt_alloc_from_slice(rt_ctx* ctx, int32_t dtype, const void* host_src, uint64_t len, void** out);
/* Drop of Backend::Buf: returns the block to the context's caching allocator (stream ordered). */
int32_t rt_free(rt_ctx* ctx, void* buf);
/* Backend::copy_from_slice: lengths must match (RT_E_SIZE_MISMATCH otherwise). */
int32_t rt_copy_from_slice(rt_ctx* ctx, int32_t dtype, void* dst, uint64_t dst_len, const void* host_src, uint64_t src_len);
/* Backend::copy_range_within: device-to-device copy of `len` elements.  A range copied onto itself is a no-op; ranges of one buffer
 * that overlap otherwise are refused with RT_E_INVALID (the trait's `&mut dst` / `&src` pair cannot express them either). */
int32_t rt_copy_range_within(rt_ctx* ctx, int32_t dtype, void* dst, uint64_t dst_len, const void* src, uint64_t src_len,
                             uint64_t dst_offset, uint64_t src_offset, uint64_t len);
/* Backend::read / Backend::write: one element; synchronises first. */
int32_t rt_read(rt_ctx* ctx, int32_t dtype, const void* buf, uint64_t buf_len, uint64_t offset, void* out_value);
int32_t rt_write(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, uint64_t offset, const void* value);
/* Backend::copy: fresh buffer holding a copy of `src`. */
int32_t rt_copy(rt_ctx* ctx, int32_t dtype, const void* src, uint64_t len, void** out);
/* Backend::dump: download the whole buffer into `host_dst` (len elements); synchronises. */
int32_t rt_dump(rt_ctx* ctx, int32_t dtype, const void* src, uint64_t len, void* host_dst);
/* PartialEq of Backend::Buf (backend/cuda.rs:59-141): lengths equal and all elements `==` (NaN != NaN). */
int32_t rt_equal(rt_ctx* ctx, int32_t dtype, const void* a, uint64_t a_len, const void* b, uint64_t b_len, int32_t* out_equal);
/* Backend::convert: elementwise dtype conversion between equally long buffers (core/value.rs:255-462), every pair of the 13 dtypes:
 * Rust `as` between integers, float -> integer rounds half away from zero and saturates (NaN -> 0), integer -> float rounds to
 * nearest (u128 -> f32 overflows to +inf), anything -> bool is x != 0. */
int32_t rt_convert(rt_ctx* ctx, int32_t src_dtype, const void* src, uint64_t src_len, int32_t dst_dtype, void* dst, uint64_t dst_len);

/* ---- fill (Backend::fill_contiguous / fill_1d_strided / fill_nd, backend/mod.rs:270-294) ----------------------- */
int32_t rt_fill_contiguous(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value, uint64_t start, uint64_t len);
int32_t rt_fill_1d_strided(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value,
                           uint64_t offset, int64_t stride, uint64_t len);
int32_t rt_fill_nd(rt_ctx* ctx, int32_t dtype, void* buf, uint64_t buf_len, const void* value,
                   uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides);

/* ---- in-place unary ops (Backend::apply_<op>_{contiguous,1d_strided,nd}, backend/mod.rs:96-141, 311-355) ------ */
/* The exact ops (neg, relu, abs, sqrt, reciprocal, square, cube, sign, the four roundings) give the bits of the reference's Cpu
 * backend.  The transcendental ops are within the reference's own test tolerance of 1e-5 but not bit-identical to the platform
 * libm it calls.  Where the backend computes by its own routine instead of the device library's the bound is, in units of the last
 * place of the exact value: f64 ln and ln1p 1, f64 asin 2, f64 acos 1.5, f64 tan 3 (arguments below 2^30; the library routine
 * beyond), f32 ln1p 3.5.  f64 sigmoid, silu, tanh, sinh, cosh, asinh, acosh, atanh and the log(base) / log1p(base) scalar ops are
 * the reference's formulas over these routines and the library's exponential, with quotients and square roots that are within an
 * ulp instead of correctly rounded; at the ends of their ranges (overflow, +-1, +-inf, NaN) they return what the formulas return. */
int32_t rt_unary_contiguous(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, uint64_t start, uint64_t len);
int32_t rt_unary_1d_strided(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len,
                            uint64_t offset, int64_t stride, uint64_t len);
int32_t rt_unary_nd(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len,
                    uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides);

/* ---- in-place scalar ops (Backend::scalar_apply_<op>_{...}, backend/mod.rs:143-213, 327-334) ----------------- */
int32_t rt_scalar_contiguous(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, const void* value,
                             uint64_t start, uint64_t len);
int32_t rt_scalar_1d_strided(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, const void* value,
                             uint64_t offset, int64_t stride, uint64_t len);
int32_t rt_scalar_nd(rt_ctx* ctx, int32_t dtype, int32_t op, void* buf, uint64_t buf_len, const void* value,
                     uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides);

/* ---- N-d broadcast (Backend::broadcast, backend/mod.rs:296-309; Cpu backend/cpu.rs:292-352) --------------------
 * dst[c] = left[c] (op) right[c] for every coordinate c of `shape`.  The three operands share `shape`
 * (expansion is expressed as stride 0, ops/broadcast/mod.rs:13-55); strides may be negative.  dst may be the
 * very same view as an input (same buffer, offset and strides: the in-place `a op= b`).  A destination whose address range meets
 * an input's in any other way is refused with RT_E_INVALID: block order would decide the result.
 * Integer division: a zero divisor or MIN / -1 inside the tensors (a panic in the reference, ops/base.rs:27-37) cannot be seen
 * before the kernel has run; the kernel stores 0 / MIN for such elements and sets a fault word of the context, and the next
 * call that waits for the stream (rt_sync, rt_read, rt_dump, rt_equal) returns RT_E_ARITH once and clears it.  The same holds for
 * rt_scalar_* division of a signed tensor by -1.  A zero scalar divisor is refused at once.
 * Device memory: an input of 256 KiB and more that is a permuted view with short contiguous pieces (it steps 64 bytes or more along
 * dst's inner dim, or its unit-stride rows are shorter than 256 bytes and lie scattered) may first be copied into a row-major
 * temporary of its own size, taken from and returned to the context's block cache like an rt_alloc_uninit / rt_free pair -- not
 * when dst and the other input are row-major runs of f32, f64 or 32- / 64-bit integers under + - * (floats also /), which one
 * kernel handles.  If the block cannot be had the op runs without it, slower.  No other input layout makes this call allocate. */
int32_t rt_broadcast(rt_ctx* ctx, int32_t dtype, int32_t op, int32_t rank, const uint64_t* shape,
                     const void* left, uint64_t left_len, uint64_t left_offset, const int64_t* left_strides,
                     const void* right, uint64_t right_len, uint64_t right_offset, const int64_t* right_strides,
                     void* dst, uint64_t dst_len, uint64_t dst_offset, const int64_t* dst_strides);

/* ---- reductions (Backend::apply_reduce_contiguous_flat / _nd, backend/mod.rs:357-409; Cpu backend/cpu.rs:397-449)
 * Flat: dst[0] = fold(src[start .. start+len]).  Nd: `src` described by (offset, shape, strides) must be row-major
 * contiguous; viewed as (outer, R = shape[dim], inner), dst[o*inner + i] = fold_k src[offset + (o*R + k)*inner + i].
 * The offset is honoured (as backend/cuda.rs:1934 does; the Cpu backend drops it, backend/cpu.rs:434).
 * Float sums are tree sums: within 1e-5 (f32) / 1e-12 (f64) of sum|x| of the sequential result; integer results,
 * max and min are bit-exact.  f32/f64 as in the reference, plus the 8..64-bit integers. */
int32_t rt_reduce_flat(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len,
                       void* dst, uint64_t dst_len, uint64_t start, uint64_t len);
int32_t rt_reduce_nd(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len,
                     uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides,
                     void* dst, uint64_t dst_len, int32_t dim);
/* The same two entry points also take the statistics the reference's Cuda backend offers and its Cpu backend panics on
 * (ops/reduction/mod.rs:185; kernels K/kernels/reduction/reduce.cu:167-213 variance, 641-735 logsumexp, 66-97 norms), f32/f64 only:
 *   RT_R_VARIANCE [| RT_R_FLAG_UNBIASED] [| RT_R_FLAG_STD]   m2 / (n - 1 | n), m2 = sum (x - mean)^2 merged pairwise
 *                                                           (Chan's update, never sum x^2 - n mean^2); n = 1 unbiased gives NaN
 *   RT_R_LOGSUMEXP                                           max + log(sum exp(x - max)); -inf for an empty or all -inf run, +inf
 *                                                           when +inf occurs (the reference's flat launcher has no case for it
 *                                                           and leaves dst unwritten, reduce.cu:795-832; here flat works too)
 *   RT_R_NORM | RT_R_FLAG_L1 / RT_R_FLAG_L2                  sum |x| / sqrt(sum x^2)
 * Results are within 1e-5 (f32) / 1e-12 (f64), relative, of the same quantity accumulated in higher precision (variance: times its
 * condition number sqrt(1 + mean^2 / var); logsumexp: relative to max(|result|, |largest element|), the two terms it adds).
 * The exponentials of the logsumexp terms: the hardware's for f32 (a few ulp), for f64 a routine written for arguments <= 0, within
 * 1.5 ulp; a NaN element gives NaN, whatever else the run holds.
 * Float max / min return the sequential loop's result bit for bit, the sign of a zero result included (the first zero of the run).
 * RT_R_ARGMAX / RT_R_ARGMIN are refused here with RT_E_INVALID (kinds cannot be swapped between entry points,
 * backend/remote/remote_tests.rs:857-859). */

/* Backend::apply_argmax_contiguous_flat / apply_argmax_contiguous_nd (backend/mod.rs:412-463; the Cpu backend has todo!() there,
 * backend/cpu.rs:451-471; Cuda: reduce.cu:843-990).  dst holds u64 indices: for the flat form the position inside the run
 * (0 = element `start`), for the nd form the coordinate along `dim` of each of the outer * inner outputs.  The smallest index of
 * the extremum wins; NaN never wins; 0 for an empty run and when no element beats the starting value (T::MIN / T::MAX, as in
 * the reference's kernel).  op is RT_R_ARGMAX or RT_R_ARGMIN, anything else is RT_E_INVALID.  f32/f64 as in the reference, plus
 * the 8..64-bit integers.  Same validation as rt_reduce_flat / rt_reduce_nd. */
int32_t rt_argmax_flat(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len,
                       uint64_t* dst, uint64_t dst_len, uint64_t start, uint64_t len);
int32_t rt_argmax_nd(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len,
                     uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides,
                     uint64_t* dst, uint64_t dst_len, int32_t dim);

/* ---- reduction that allocates nothing -----------------------------------------------------------------------------------
 * No counterpart in the reference.  For callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  Same arguments, validation, kernels and results (bit for bit) as rt_reduce_nd, but the
 * partial results of a split reduction go to a workspace of RT_STATIC_SCRATCH_BYTES that is part of the library's device image
 * (every device the library runs on holds it until the process ends) instead of the context's on-demand scratch buffer; the call
 * performs no hipMalloc / hipFree.  A reduction whose partials do not fit is refused with RT_E_INVALID before anything is launched
 * (partials = splits * outer * inner elements: sum / prod / max / min / mean of any shape stay below 1 MiB, e.g. 512 KiB for the
 * axis-0 sum of (8192, 32768) f32; the statistics keep states of 8 .. 24 bytes per partial and can exceed it when many columns are
 * split).  All calls on one device share the workspace: calls that overlap on one device (two contexts) race on it. */
#define RT_STATIC_SCRATCH_BYTES (1u << 20)
int32_t rt_reduce_nd_static(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len,
                            uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides,
                            void* dst, uint64_t dst_len, int32_t dim);

/* ---- out-of-place unary / scalar ops ---------------------------------------------------------------------------------
 * dst[0 .. len) = op(src[start .. start + len)); the source is only read.  The trait has in-place ops only: `tensor.relu()`,
 * `tensor * 3.0` and the other value-returning forms clone the tensor and then run the in-place op (ops/unary/mod.rs:114-126,
 * ops/scalar/add.rs:93-97), i.e. 4 * N * sizeof(T) of traffic in two passes.  These two entry points give the same result in
 * one pass over 2 * N * sizeof(T) for a contiguous source (gather other views first); op codes, dtype rules and errors are
 * those of rt_unary_* / rt_scalar_*.  RT_E_WRONG_DIMS is never returned here (the run is contiguous by construction);
 * RT_E_OUT_OF_BOUNDS when the run leaves src or len exceeds dst_len. */
int32_t rt_unary_to(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, uint64_t start, uint64_t len,
                    void* dst, uint64_t dst_len);
int32_t rt_scalar_to(rt_ctx* ctx, int32_t dtype, int32_t op, const void* src, uint64_t src_len, const void* value,
                     uint64_t start, uint64_t len, void* dst, uint64_t dst_len);

/* ---- fused passes of the broadcast / reduce training step ------------------------------------------------------------------
 * No single counterpart in the trait: the reference's engine issues y = relu(x + bias), loss = mean_l1_loss(y, target)
 * (ops/broadcast/l1.rs:49-84) and its backward (grad/backwards.rs:148-161, 229-239, 516-538) as one backend call per arithmetic
 * step, with a full-size temporary between each two.  These three optional entry points run the same IEEE operations per element,
 * in the same order, in one pass each; every element-wise result is bit for bit what the separate calls give, the two sums are tree
 * sums within the tolerance of rt_reduce_*.  f32 / f64, row-major contiguous operands from element 0 of 16-byte aligned buffers,
 * cols (resp. n) a whole number of 16-byte vectors -- anything else is RT_E_INVALID and the caller issues the separate ops.
 *   rt_fused_bias_relu          y[i, j] = relu(x[i, j] + bias[j])
 *   rt_fused_l1_forward         gmap[k] = sign(y[k] - target[k]) / N,  loss[0] = (sum_k |y[k] - target[k]|) / N,  N = (T)(f32)n
 *   rt_fused_l1_relu_backward   dbias[j] = sum_i (y[i, j] > 0 ? 1 : 0) * (gmap[i, j] * upstream[0])   (upstream: one device element,
 *                               the loss-seeded root of grad/mod.rs:442-447 or a one)
 * y may be x itself and gmap may be y or target itself (in place); an output that overlaps an input in any other way is RT_E_INVALID. */
int32_t rt_fused_bias_relu(rt_ctx* ctx, int32_t dtype, const void* x, uint64_t x_len, const void* bias, uint64_t bias_len,
                           void* y, uint64_t y_len, uint64_t rows, uint64_t cols);
int32_t rt_fused_l1_forward(rt_ctx* ctx, int32_t dtype, const void* y, uint64_t y_len, const void* target, uint64_t target_len,
                            void* gmap, uint64_t gmap_len, void* loss, uint64_t loss_len, uint64_t n);
int32_t rt_fused_l1_relu_backward(rt_ctx* ctx, int32_t dtype, const void* gmap, uint64_t gmap_len, const void* y, uint64_t y_len,
                                  const void* upstream, uint64_t upstream_len, void* dbias, uint64_t dbias_len, uint64_t rows, uint64_t cols);
/* The same step without the gradient map, which is a temporary of the tape and not a result (5 instead of 7 passes over a tensor):
 *   rt_fused_bias_relu_l1         y[i, j] = relu(x[i, j] + bias[j]),  loss[0] = (sum |y - target|) / N      (reads x, target; writes y)
 *   rt_fused_l1_relu_backward_t   dbias[j] = sum_i (y[i, j] > 0 ? 1 : 0) * ((sign(y[i, j] - target[i, j]) / N) * upstream[0])
 * with N = (T)(f32)(rows * cols).  Per element these are the operations of the three-pass form in the same order, so y and every
 * summand are bit for bit the same; same operand requirements; y may be x itself. */
int32_t rt_fused_bias_relu_l1(rt_ctx* ctx, int32_t dtype, const void* x, uint64_t x_len, const void* bias, uint64_t bias_len,
                              const void* target, uint64_t target_len, void* y, uint64_t y_len, void* loss, uint64_t loss_len,
                              uint64_t rows, uint64_t cols);
int32_t rt_fused_l1_relu_backward_t(rt_ctx* ctx, int32_t dtype, const void* y, uint64_t y_len, const void* target, uint64_t target_len,
                                    const void* upstream, uint64_t upstream_len, void* dbias, uint64_t dbias_len, uint64_t rows, uint64_t cols);

/* ---- fused elementwise chain ------------------------------------------------------------------------------------------------
 * No single counterpart in the trait: the reference issues an expression such as `c = relu(a * 3.0 + b); c -= 1.0` as one backend
 * call per operator, each a pass over the whole tensor, with a clone before every value-returning scalar / unary op
 * (ops/scalar/add.rs:84-113, ops/unary/mod.rs:114-126).  This entry point runs a program of up to RT_CHAIN_MAX_STEPS such steps in
 * registers, reading each input once and writing the result once:
 *     acc = inputs[0][input_starts[0] + i];  for every step: acc = step(acc);  dst[dst_start + i] = acc        (i < len)
 *   RT_CHAIN_UNARY       acc = op(acc)                       op: rt_unary_op
 *   RT_CHAIN_SCALAR      acc = acc op value                  op: rt_scalar_op, value: one element of dtype
 *   RT_CHAIN_BINARY      acc = acc op inputs[operand][..]    op: rt_binary_op
 *   RT_CHAIN_BINARY_REV  acc = inputs[operand][..] op acc
 * Each step is the same IEEE / wrapping operation as the separate call, in the same order (no contraction), so the result is bit for
 * bit that of the sequence.  All operands are forward contiguous runs of `len` elements (gather other views first), in any alignment.
 * dst may be the very run of one of the inputs (in place); any other overlap is RT_E_INVALID.  Available: f32 / f64 and the 8..64-bit
 * integers; unary relu abs step (+ neg abs_grad for signed and float; + sqrt floor ceil round trunc rsqrt reciprocal square cube sign
 * exp sigmoid silu tanh for float), scalar add sub mul leaky_relu leaky_grad (+ div for float), binary add sub mul (+ div for float).
 * Anything else is RT_E_DTYPE and the caller issues the separate ops (integer division reports its faults per launch; the other float
 * ops are ALU-bound on their own). */
#define RT_CHAIN_MAX_STEPS 8
#define RT_CHAIN_MAX_INPUTS 4
typedef enum rt_chain_kind { RT_CHAIN_UNARY = 0, RT_CHAIN_SCALAR = 1, RT_CHAIN_BINARY = 2, RT_CHAIN_BINARY_REV = 3 } rt_chain_kind;
typedef struct rt_chain_step {
    int32_t kind;        /* rt_chain_kind */
    int32_t op;          /* rt_unary_op / rt_scalar_op / rt_binary_op according to kind */
    int32_t operand;     /* binary kinds: index into inputs[] of the other side */
    int32_t reserved;    /* 0 */
    uint8_t value[8];    /* scalar kind: the element, in the dtype's own representation */
} rt_chain_step;
int32_t rt_fused_chain(rt_ctx* ctx, int32_t dtype, int32_t n_inputs, const void* const* inputs, const uint64_t* input_lens,
                       const uint64_t* input_starts, uint64_t len, int32_t n_steps, const rt_chain_step* steps,
                       void* dst, uint64_t dst_len, uint64_t dst_start);

/* ---- matmul ------------------------------------------------------------------------------------------------------
 * BackendMatMul::matmul (backend/mod.rs:474-485; Cpu backend/cpu.rs:725-951), argument list of protocol Op::Matmul
 * (backend/remote/protocol.rs:269-277): dst[b] = lhs[b] (m x k) * rhs[b] (k x n) for every batch, dst row-major and
 * contiguous from element 0 (b*m*n elements).  Each operand comes with its meta and the layout the caller found for its
 * last two dims (core/meta.rs:744-750, ops/linalg/matmul.rs:200-251): row-major = column stride 1, column-major = row
 * stride 1; batch dims must collapse into one stride; strides must not be negative.  The checks are those of
 * backend/remote/server.rs:299-334 and 605-636 (RT_E_INVALID / RT_E_OUT_OF_BOUNDS); dst must not be one of the inputs.
 * f32/f64 run on rocBLAS (loaded on first use), every other dtype -- all 13 are accepted, as the Cpu backend's generic
 * loop does -- on a tiled kernel with the reference's wrapping `sum += a * b`.  Mixed layouts are accepted for every dtype
 * (the Cpu backend has them for f32/f64 only). */
typedef enum rt_contiguity { RT_ROW_MAJOR = 0, RT_COLUMN_MAJOR = 1, RT_CONTIGUITY_NONE = 2 } rt_contiguity;
int32_t rt_matmul(rt_ctx* ctx, int32_t dtype,
                  const void* lhs, uint64_t lhs_len, uint64_t lhs_offset, int32_t lhs_rank, const uint64_t* lhs_shape,
                  const int64_t* lhs_strides, int32_t lhs_contiguity,
                  const void* rhs, uint64_t rhs_len, uint64_t rhs_offset, int32_t rhs_rank, const uint64_t* rhs_shape,
                  const int64_t* rhs_strides, int32_t rhs_contiguity,
                  void* dst, uint64_t dst_len, uint64_t b, uint64_t m, uint64_t k, uint64_t n);

/* ---- strided gather (what TensorView::owned / contiguous need, core/tensor.rs:299-325: the reference issues one
 * copy_range_within per forward-contiguous run; this is the same result in one launch) ------------------------- */
int32_t rt_gather(rt_ctx* ctx, int32_t dtype, const void* src, uint64_t src_len, uint64_t offset, int32_t rank,
                  const uint64_t* shape, const int64_t* strides, void* dst, uint64_t dst_len);

/* ---- timing and allocator introspection (no counterpart in the reference; used by the benchmark) -------------- */
typedef struct rt_event rt_event;
int32_t rt_event_create(rt_ctx* ctx, rt_event** out);
int32_t rt_event_record(rt_ctx* ctx, rt_event* ev);              /* on the context's stream */
int32_t rt_event_elapsed_ms(rt_ctx* ctx, rt_event* start, rt_event* stop, float* out_ms);   /* waits for `stop` */
int32_t rt_event_destroy(rt_ctx* ctx, rt_event* ev);
/* bytes currently handed out, bytes cached in free lists, number of hipMalloc calls so far (blocks and growth of the scratch buffer) */
int32_t rt_mem_stats(rt_ctx* ctx, uint64_t* in_use, uint64_t* cached, uint64_t* device_allocs);
int32_t rt_mem_trim(rt_ctx* ctx);                                /* hipFree everything in the free lists */

/* ---- the host-side checks on their own (no counterpart in the reference's trait; they restate its remote server's validators,
 * backend/remote/server.rs:241-295) -------------------------------------------------------------------------------------------------
 * What every entry point does to a view before it launches anything, callable without a context or a device, so that the validation
 * can be exercised (and fuzzed under a sanitizer) on a machine without a GPU.
 *   rt_debug_check_view     the extent check (lowest and highest addressed element inside [0, len), 128-bit arithmetic) and, for a
 *                           non-empty view, the canonical layout a kernel would get: size-1 dims dropped, dims flipped to non-negative
 *                           strides, sorted by stride, adjacent dims merged.  out_shape / out_strides hold RT_MAX_RANK entries;
 *                           RT_E_RANK when more dims remain.  *out_count = number of elements (0 for an empty view).
 *   rt_debug_check_overlap  two views of one buffer with a common shape: *out_meet = their address ranges intersect, *out_same = they
 *                           are the very same view (the one aliasing an output may have with an input). */
int32_t rt_debug_check_view(uint64_t offset, int32_t rank, const uint64_t* shape, const int64_t* strides, uint64_t len,
                            uint64_t* out_count, int32_t* out_rank, int64_t* out_shape, int64_t* out_strides, int64_t* out_offset);
int32_t rt_debug_check_overlap(int32_t elem_size, int32_t rank, const uint64_t* shape, uint64_t a_offset, const int64_t* a_strides,
                               uint64_t b_offset, const int64_t* b_strides, uint64_t len, int32_t* out_meet, int32_t* out_same);

#ifdef __cplusplus
}
#endif
#endif /* RT_HIP_H */

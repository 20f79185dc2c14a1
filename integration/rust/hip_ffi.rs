//! `extern "C"` declarations of librt_hip.so, one per entry point of include/rt_hip.h (same names, same argument order).
//! Goes to `libs/rtensors/src/backend/hip_ffi.rs`.  Written by hand against the header: the ABI is plain pointers and
//! integers, so no bindgen step is needed.  `tests/test_rust_binding.py` checks names and argument counts against the header.
#![allow(non_camel_case_types, dead_code)]

use std::os::raw::{c_char, c_void};

/// Opaque context: device + stream + caching allocator.
#[repr(C)]
pub struct rt_ctx {
    _private: [u8; 0],
}
/// Opaque timing event.
#[repr(C)]
pub struct rt_event {
    _private: [u8; 0],
}

/// One step of a fused elementwise chain (`rt_chain_step`): 24 bytes, same field order as the header.
#[repr(C)]
#[derive(Clone, Copy, Debug, Default)]
pub struct rt_chain_step {
    pub kind: i32,
    pub op: i32,
    pub operand: i32,
    pub reserved: i32,
    pub value: [u8; 8],
}

// rt_chain_kind and the limits of a chain
pub const RT_CHAIN_UNARY: i32 = 0;
pub const RT_CHAIN_SCALAR: i32 = 1;
pub const RT_CHAIN_BINARY: i32 = 2;
pub const RT_CHAIN_BINARY_REV: i32 = 3;
pub const RT_CHAIN_MAX_STEPS: i32 = 8;
pub const RT_CHAIN_MAX_INPUTS: i32 = 4;

// rt_status
pub const RT_OK: i32 = 0;
pub const RT_E_INVALID: i32 = 1;
pub const RT_E_DTYPE: i32 = 2;
pub const RT_E_OUT_OF_BOUNDS: i32 = 3;
pub const RT_E_HIP: i32 = 4;
pub const RT_E_OOM: i32 = 5;
pub const RT_E_RANK: i32 = 6;
pub const RT_E_ARITH: i32 = 7;
pub const RT_E_WRONG_DIMS: i32 = 8;
pub const RT_E_SIZE_MISMATCH: i32 = 9;

// rt_unary_op: declaration order of protocol::UnaryOp, then the two gradient maps
pub const RT_U_NEG: i32 = 0;
pub const RT_U_RELU: i32 = 1;
pub const RT_U_SIGMOID: i32 = 2;
pub const RT_U_SILU: i32 = 3;
pub const RT_U_TANH: i32 = 4;
pub const RT_U_ABS: i32 = 5;
pub const RT_U_SQRT: i32 = 6;
pub const RT_U_LN: i32 = 7;
pub const RT_U_EXPM1: i32 = 8;
pub const RT_U_LN1P: i32 = 9;
pub const RT_U_FLOOR: i32 = 10;
pub const RT_U_CEIL: i32 = 11;
pub const RT_U_ROUND: i32 = 12;
pub const RT_U_TRUNC: i32 = 13;
pub const RT_U_SIN: i32 = 14;
pub const RT_U_COS: i32 = 15;
pub const RT_U_TAN: i32 = 16;
pub const RT_U_ASIN: i32 = 17;
pub const RT_U_ACOS: i32 = 18;
pub const RT_U_ATAN: i32 = 19;
pub const RT_U_SINH: i32 = 20;
pub const RT_U_COSH: i32 = 21;
pub const RT_U_ASINH: i32 = 22;
pub const RT_U_ACOSH: i32 = 23;
pub const RT_U_ATANH: i32 = 24;
pub const RT_U_RSQRT: i32 = 25;
pub const RT_U_RECIPROCAL: i32 = 26;
pub const RT_U_SQUARE: i32 = 27;
pub const RT_U_CUBE: i32 = 28;
pub const RT_U_EXP: i32 = 29;
pub const RT_U_SIGN: i32 = 30;
pub const RT_U_STEP: i32 = 31;
pub const RT_U_ABS_GRAD: i32 = 32;

// rt_scalar_op: declaration order of protocol::ScalarOp, then the leaky-ReLU gradient map
pub const RT_S_ADD: i32 = 0;
pub const RT_S_SUB: i32 = 1;
pub const RT_S_MUL: i32 = 2;
pub const RT_S_DIV: i32 = 3;
pub const RT_S_LOG: i32 = 4;
pub const RT_S_LOG1P: i32 = 5;
pub const RT_S_LEAKY_RELU: i32 = 6;
pub const RT_S_ELU: i32 = 7;
pub const RT_S_LEAKY_GRAD: i32 = 8;

// flag bits on top of ReductionOpTypes::get_code()
pub const RT_R_FLAG_UNBIASED: i32 = 0x100;
pub const RT_R_FLAG_STD: i32 = 0x200;
pub const RT_R_FLAG_L1: i32 = 0x100;
pub const RT_R_FLAG_L2: i32 = 0x200;

// rt_contiguity
pub const RT_ROW_MAJOR: i32 = 0;
pub const RT_COLUMN_MAJOR: i32 = 1;
pub const RT_CONTIGUITY_NONE: i32 = 2;

pub const RT_STATIC_SCRATCH_BYTES: u32 = 1 << 20;

#[link(name = "rt_hip")]
extern "C" {
    pub fn rt_ctx_create(device: i32, out: *mut *mut rt_ctx) -> i32;
    pub fn rt_ctx_destroy(ctx: *mut rt_ctx) -> i32;
    pub fn rt_sync(ctx: *mut rt_ctx) -> i32;
    pub fn rt_last_error() -> *const c_char;
    pub fn rt_status_name(status: i32) -> *const c_char;
    pub fn rt_dtype_size(dtype: i32) -> i32;
    pub fn rt_device_count(out: *mut i32) -> i32;
    pub fn rt_alloc(ctx: *mut rt_ctx, dtype: i32, len: u64, out: *mut *mut c_void) -> i32;
    pub fn rt_alloc_uninit(ctx: *mut rt_ctx, dtype: i32, len: u64, out: *mut *mut c_void) -> i32;
    pub fn rt_alloc_from_slice(ctx: *mut rt_ctx, dtype: i32, host_src: *const c_void, len: u64, out: *mut *mut c_void) -> i32;
    pub fn rt_free(ctx: *mut rt_ctx, buf: *mut c_void) -> i32;
    pub fn rt_copy_from_slice(ctx: *mut rt_ctx, dtype: i32, dst: *mut c_void, dst_len: u64, host_src: *const c_void,
                              src_len: u64) -> i32;
    pub fn rt_copy_range_within(ctx: *mut rt_ctx, dtype: i32, dst: *mut c_void, dst_len: u64, src: *const c_void,
                                src_len: u64, dst_offset: u64, src_offset: u64, len: u64) -> i32;
    pub fn rt_read(ctx: *mut rt_ctx, dtype: i32, buf: *const c_void, buf_len: u64, offset: u64, out_value: *mut c_void) -> i32;
    pub fn rt_write(ctx: *mut rt_ctx, dtype: i32, buf: *mut c_void, buf_len: u64, offset: u64, value: *const c_void) -> i32;
    pub fn rt_copy(ctx: *mut rt_ctx, dtype: i32, src: *const c_void, len: u64, out: *mut *mut c_void) -> i32;
    pub fn rt_dump(ctx: *mut rt_ctx, dtype: i32, src: *const c_void, len: u64, host_dst: *mut c_void) -> i32;
    pub fn rt_equal(ctx: *mut rt_ctx, dtype: i32, a: *const c_void, a_len: u64, b: *const c_void, b_len: u64,
                    out_equal: *mut i32) -> i32;
    pub fn rt_convert(ctx: *mut rt_ctx, src_dtype: i32, src: *const c_void, src_len: u64, dst_dtype: i32, dst: *mut c_void,
                      dst_len: u64) -> i32;
    pub fn rt_fill_contiguous(ctx: *mut rt_ctx, dtype: i32, buf: *mut c_void, buf_len: u64, value: *const c_void, start: u64,
                              len: u64) -> i32;
    pub fn rt_fill_1d_strided(ctx: *mut rt_ctx, dtype: i32, buf: *mut c_void, buf_len: u64, value: *const c_void,
                              offset: u64, stride: i64, len: u64) -> i32;
    pub fn rt_fill_nd(ctx: *mut rt_ctx, dtype: i32, buf: *mut c_void, buf_len: u64, value: *const c_void, offset: u64,
                      rank: i32, shape: *const u64, strides: *const i64) -> i32;
    pub fn rt_unary_contiguous(ctx: *mut rt_ctx, dtype: i32, op: i32, buf: *mut c_void, buf_len: u64, start: u64, len: u64) -> i32;
    pub fn rt_unary_1d_strided(ctx: *mut rt_ctx, dtype: i32, op: i32, buf: *mut c_void, buf_len: u64, offset: u64,
                               stride: i64, len: u64) -> i32;
    pub fn rt_unary_nd(ctx: *mut rt_ctx, dtype: i32, op: i32, buf: *mut c_void, buf_len: u64, offset: u64, rank: i32,
                       shape: *const u64, strides: *const i64) -> i32;
    pub fn rt_scalar_contiguous(ctx: *mut rt_ctx, dtype: i32, op: i32, buf: *mut c_void, buf_len: u64, value: *const c_void,
                                start: u64, len: u64) -> i32;
    pub fn rt_scalar_1d_strided(ctx: *mut rt_ctx, dtype: i32, op: i32, buf: *mut c_void, buf_len: u64, value: *const c_void,
                                offset: u64, stride: i64, len: u64) -> i32;
    pub fn rt_scalar_nd(ctx: *mut rt_ctx, dtype: i32, op: i32, buf: *mut c_void, buf_len: u64, value: *const c_void,
                        offset: u64, rank: i32, shape: *const u64, strides: *const i64) -> i32;
    pub fn rt_broadcast(ctx: *mut rt_ctx, dtype: i32, op: i32, rank: i32, shape: *const u64, left: *const c_void,
                        left_len: u64, left_offset: u64, left_strides: *const i64, right: *const c_void, right_len: u64,
                        right_offset: u64, right_strides: *const i64, dst: *mut c_void, dst_len: u64, dst_offset: u64,
                        dst_strides: *const i64) -> i32;
    pub fn rt_reduce_flat(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, dst: *mut c_void,
                          dst_len: u64, start: u64, len: u64) -> i32;
    pub fn rt_reduce_nd(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, offset: u64, rank: i32,
                        shape: *const u64, strides: *const i64, dst: *mut c_void, dst_len: u64, dim: i32) -> i32;
    pub fn rt_argmax_flat(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, dst: *mut u64,
                          dst_len: u64, start: u64, len: u64) -> i32;
    pub fn rt_argmax_nd(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, offset: u64, rank: i32,
                        shape: *const u64, strides: *const i64, dst: *mut u64, dst_len: u64, dim: i32) -> i32;
    pub fn rt_reduce_nd_static(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, offset: u64,
                               rank: i32, shape: *const u64, strides: *const i64, dst: *mut c_void, dst_len: u64, dim: i32) -> i32;
    pub fn rt_unary_to(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, start: u64, len: u64,
                       dst: *mut c_void, dst_len: u64) -> i32;
    pub fn rt_scalar_to(ctx: *mut rt_ctx, dtype: i32, op: i32, src: *const c_void, src_len: u64, value: *const c_void,
                        start: u64, len: u64, dst: *mut c_void, dst_len: u64) -> i32;
    pub fn rt_fused_bias_relu(ctx: *mut rt_ctx, dtype: i32, x: *const c_void, x_len: u64, bias: *const c_void, bias_len: u64,
                              y: *mut c_void, y_len: u64, rows: u64, cols: u64) -> i32;
    pub fn rt_fused_l1_forward(ctx: *mut rt_ctx, dtype: i32, y: *const c_void, y_len: u64, target: *const c_void,
                               target_len: u64, gmap: *mut c_void, gmap_len: u64, loss: *mut c_void, loss_len: u64, n: u64) -> i32;
    pub fn rt_fused_l1_relu_backward(ctx: *mut rt_ctx, dtype: i32, gmap: *const c_void, gmap_len: u64, y: *const c_void,
                                     y_len: u64, upstream: *const c_void, upstream_len: u64, dbias: *mut c_void,
                                     dbias_len: u64, rows: u64, cols: u64) -> i32;
    pub fn rt_fused_bias_relu_l1(ctx: *mut rt_ctx, dtype: i32, x: *const c_void, x_len: u64, bias: *const c_void, bias_len: u64,
                                 target: *const c_void, target_len: u64, y: *mut c_void, y_len: u64, loss: *mut c_void, loss_len: u64,
                                 rows: u64, cols: u64) -> i32;
    pub fn rt_fused_l1_relu_backward_t(ctx: *mut rt_ctx, dtype: i32, y: *const c_void, y_len: u64, target: *const c_void,
                                       target_len: u64, upstream: *const c_void, upstream_len: u64, dbias: *mut c_void,
                                       dbias_len: u64, rows: u64, cols: u64) -> i32;
    pub fn rt_fused_chain(ctx: *mut rt_ctx, dtype: i32, n_inputs: i32, inputs: *const *const c_void, input_lens: *const u64,
                          input_starts: *const u64, len: u64, n_steps: i32, steps: *const rt_chain_step, dst: *mut c_void,
                          dst_len: u64, dst_start: u64) -> i32;
    pub fn rt_matmul(ctx: *mut rt_ctx, dtype: i32, lhs: *const c_void, lhs_len: u64, lhs_offset: u64, lhs_rank: i32,
                     lhs_shape: *const u64, lhs_strides: *const i64, lhs_contiguity: i32, rhs: *const c_void, rhs_len: u64,
                     rhs_offset: u64, rhs_rank: i32, rhs_shape: *const u64, rhs_strides: *const i64, rhs_contiguity: i32,
                     dst: *mut c_void, dst_len: u64, b: u64, m: u64, k: u64, n: u64) -> i32;
    pub fn rt_gather(ctx: *mut rt_ctx, dtype: i32, src: *const c_void, src_len: u64, offset: u64, rank: i32,
                     shape: *const u64, strides: *const i64, dst: *mut c_void, dst_len: u64) -> i32;
    pub fn rt_debug_check_view(offset: u64, rank: i32, shape: *const u64, strides: *const i64, len: u64, out_count: *mut u64,
                               out_rank: *mut i32, out_shape: *mut i64, out_strides: *mut i64, out_offset: *mut i64) -> i32;
    pub fn rt_debug_check_overlap(elem_size: i32, rank: i32, shape: *const u64, a_offset: u64, a_strides: *const i64,
                                  b_offset: u64, b_strides: *const i64, len: u64, out_meet: *mut i32, out_same: *mut i32) -> i32;
    pub fn rt_event_create(ctx: *mut rt_ctx, out: *mut *mut rt_event) -> i32;
    pub fn rt_event_record(ctx: *mut rt_ctx, ev: *mut rt_event) -> i32;
    pub fn rt_event_elapsed_ms(ctx: *mut rt_ctx, start: *mut rt_event, stop: *mut rt_event, out_ms: *mut f32) -> i32;
    pub fn rt_event_destroy(ctx: *mut rt_ctx, ev: *mut rt_event) -> i32;
    pub fn rt_mem_stats(ctx: *mut rt_ctx, in_use: *mut u64, cached: *mut u64, device_allocs: *mut u64) -> i32;
    pub fn rt_mem_trim(ctx: *mut rt_ctx) -> i32;
}

//! `Hip`: the MI355X backend behind `trait Backend` (backend/mod.rs:216-472) and `BackendMatMul` (backend/mod.rs:474-485).
//! Goes to `libs/rtensors/src/backend/hip.rs`, next to `hip_ffi.rs`, behind the cargo feature `hip`.
//!
//! Every method is one call into librt_hip.so.  The library validates each descriptor and answers with a status
//! instead of aborting, so nothing here repeats its checks; `check` turns a status into the matching `TensorError`.
//! Launches are asynchronous on the context's stream.  `read`, `dump`, `copy_from_slice` and `PartialEq` wait for it,
//! so the `dirty` flag that backend/cuda.rs:164-185 keeps on the Rust side has no counterpart here.
//!
//! `Shape` is `Vec<usize>` and `Strides` is `Vec<isize>` (core/meta.rs:12,78); both are 64 bits wide on every target
//! this backend runs on (checked at compile time below), so they go down as `*const u64` / `*const i64` without a copy.

use std::ffi::{c_void, CStr};
use std::marker::PhantomData;
use std::sync::{Arc, OnceLock};

use paste::paste;

use crate::backend::hip_ffi as ffi;
use crate::backend::{Backend, BackendMatMul};
use crate::core::meta::ContiguityTypes;
use crate::core::primitives::DeviceType;
use crate::core::primops::{Exp, InvExp, SquareRoot};
use crate::core::tensor::TensorError;
use crate::core::value::{TensorValue, WeightValue};
use crate::core::{Dim, MetaTensor};
use crate::ops::base::BinaryOpType;
use crate::ops::linalg::ConvConfig2D;
use crate::ops::reduction::{NormType, ReductionOpTypes};

const _: () = assert!(std::mem::size_of::<usize>() == 8 && std::mem::size_of::<isize>() == 8);

/// Owner of one `rt_ctx` (device, stream, caching allocator).  The library serialises calls per context.
#[derive(Debug)]
struct Ctx {
    raw: *mut ffi::rt_ctx,
    device: usize,
}
unsafe impl Send for Ctx {}
unsafe impl Sync for Ctx {}

impl Drop for Ctx {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { ffi::rt_ctx_destroy(self.raw) };
        }
    }
}

/// Text of the calling thread's last library error.
fn last_error() -> String {
    let p = unsafe { ffi::rt_last_error() };
    if p.is_null() {
        return String::new();
    }
    unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned()
}

/// Status -> `TensorError`, the one place where the two vocabularies meet.
fn check(status: i32) -> Result<(), TensorError> {
    if status == ffi::RT_OK {
        return Ok(());
    }
    let msg = last_error();
    Err(match status {
        ffi::RT_E_OUT_OF_BOUNDS => TensorError::IdxOutOfBounds(msg),
        ffi::RT_E_WRONG_DIMS | ffi::RT_E_RANK => TensorError::WrongDims(msg),
        ffi::RT_E_SIZE_MISMATCH => TensorError::SizeMismatch(msg),
        ffi::RT_E_DTYPE => TensorError::UnsupportedOperation(msg),
        ffi::RT_E_INVALID => TensorError::BackendError(msg),
        // integer division by zero (or MIN / -1) seen by a kernel since the last synchronising call
        ffi::RT_E_ARITH => TensorError::BackendError(format!("integer division fault: {msg}")),
        // RT_E_HIP, RT_E_OOM and anything a newer library may add
        _ => TensorError::HipError(msg),
    })
}

/// Backend handle.  Clones share one context, as `Cuda` clones share one `CudaContext` (backend/cuda.rs:38-51).
#[derive(Clone, Debug)]
pub struct Hip {
    ctx: Arc<Ctx>,
}

/// One context per device for the whole process: `Backend::new()` is called once per tensor constructor
/// (core/primitives.rs:455-506), and a context owns a stream and an allocator cache.
static CONTEXTS: OnceLock<Vec<OnceLock<Result<Arc<Ctx>, String>>>> = OnceLock::new();

impl Hip {
    /// Handle on `device`, or the library's message when the device or the library is not usable.
    pub fn construct(device: usize) -> Result<Self, TensorError> {
        let slots = CONTEXTS.get_or_init(|| {
            let mut n = 0i32;
            let count = if unsafe { ffi::rt_device_count(&mut n) } == ffi::RT_OK { n.max(0) as usize } else { 0 };
            (0..count).map(|_| OnceLock::new()).collect()
        });
        let slot = slots
            .get(device)
            .ok_or_else(|| TensorError::HipError(format!("HIP device {device} not found ({} visible)", slots.len())))?;
        let made = slot.get_or_init(|| {
            let mut raw = std::ptr::null_mut();
            let status = unsafe { ffi::rt_ctx_create(device as i32, &mut raw) };
            if status != ffi::RT_OK || raw.is_null() {
                return Err(last_error());
            }
            Ok(Arc::new(Ctx { raw, device }))
        });
        match made {
            Ok(ctx) => Ok(Hip { ctx: ctx.clone() }),
            Err(msg) => Err(TensorError::HipError(msg.clone())),
        }
    }

    /// Wait for everything queued on this backend's stream; reports a pending integer division fault.
    pub fn sync(&self) -> Result<(), TensorError> {
        check(unsafe { ffi::rt_sync(self.raw()) })
    }

    #[inline(always)]
    fn raw(&self) -> *mut ffi::rt_ctx {
        self.ctx.raw
    }

    fn wrap<T: TensorValue>(&self, ptr: *mut c_void, len: usize) -> HipBuf<T> {
        HipBuf { ptr, len, ctx: self.ctx.clone(), _elem: PhantomData }
    }
}

/// Device buffer of `len` elements of `T`.  Holds its context alive; returns its block to the allocator on drop.
#[derive(Debug)]
pub struct HipBuf<T: TensorValue> {
    pub(crate) ptr: *mut c_void,
    pub(crate) len: usize,
    ctx: Arc<Ctx>,
    _elem: PhantomData<T>,
}
unsafe impl<T: TensorValue> Send for HipBuf<T> {}
unsafe impl<T: TensorValue> Sync for HipBuf<T> {}

impl<T: TensorValue> Drop for HipBuf<T> {
    fn drop(&mut self) {
        // stream-ordered: work already queued on the buffer finishes before the block is handed out again
        unsafe { ffi::rt_free(self.ctx.raw, self.ptr) };
    }
}

/// Device-side comparison (replaces buffer_equal.cu + backend/cuda.rs:59-141).  Buffers of different length or on
/// different devices are unequal; a failed call compares unequal rather than panicking.
impl<T: TensorValue> PartialEq for HipBuf<T> {
    fn eq(&self, other: &Self) -> bool {
        if self.len != other.len || self.ctx.device != other.ctx.device {
            return false;
        }
        let mut same = 0i32;
        let status = unsafe {
            ffi::rt_equal(self.ctx.raw, dt::<T>(), self.ptr, self.len as u64, other.ptr, other.len as u64, &mut same)
        };
        status == ffi::RT_OK && same != 0
    }
}

/// dtype code of `T`: `DType` is `#[repr(C)]` with the discriminants the library uses (core/value.rs:566-581).
#[inline(always)]
fn dt<T: TensorValue>() -> i32 {
    T::DTYPE as i32
}

#[inline(always)]
fn val<T>(v: &T) -> *const c_void {
    v as *const T as *const c_void
}

/// Reduction word: `get_code()` in the low byte, the payload of Variance / Stdev / Norm in the flag bits -- the
/// three facts `populate_reduction_settings` (backend/cuda.rs:1750-1774) passes to the Cuda kernels.
fn reduce_word(op: &ReductionOpTypes) -> i32 {
    let flags = match op {
        ReductionOpTypes::Variance { unbiased } => {
            if *unbiased { ffi::RT_R_FLAG_UNBIASED } else { 0 }
        }
        ReductionOpTypes::Stdev { unbiased } => {
            ffi::RT_R_FLAG_STD | if *unbiased { ffi::RT_R_FLAG_UNBIASED } else { 0 }
        }
        ReductionOpTypes::Norm(NormType::L1) => ffi::RT_R_FLAG_L1,
        ReductionOpTypes::Norm(NormType::L2) => ffi::RT_R_FLAG_L2,
        _ => 0,
    };
    op.get_code() as i32 | flags
}

fn contiguity_code(c: &ContiguityTypes) -> i32 {
    match c {
        ContiguityTypes::RowMajor => ffi::RT_ROW_MAJOR,
        ContiguityTypes::ColumnMajor => ffi::RT_COLUMN_MAJOR,
        ContiguityTypes::None => ffi::RT_CONTIGUITY_NONE,
    }
}

/// The four methods of one unary op.  `apply_<op>` overrides the trait's default dispatch (backend/mod.rs:56-91):
/// the whole view goes down in one call and the library canonicalises it (signed strides, merged dims, contiguous
/// runs), which also covers what the default would have routed to the contiguous and 1-D entry points.
macro_rules! hip_unary {
    ($name:ident, $code:expr $(, where $($bound:tt)+)?) => {
        paste! {
            fn [<apply_ $name>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, meta: &MetaTensor) -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                check(unsafe {
                    ffi::rt_unary_nd(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, meta.offset as u64,
                        meta.rank() as i32, meta.shape.as_slice().as_ptr() as *const u64,
                        meta.strides.as_slice().as_ptr() as *const i64)
                })
            }

            fn [<apply_ $name _nd>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, offset: usize, shape: &[usize],
                stride: &[isize]) -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                if shape.len() != stride.len() {
                    return Err(TensorError::WrongDims(format!("shape has {} dims, strides {}", shape.len(), stride.len())));
                }
                check(unsafe {
                    ffi::rt_unary_nd(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, offset as u64,
                        shape.len() as i32, shape.as_ptr() as *const u64, stride.as_ptr() as *const i64)
                })
            }

            fn [<apply_ $name _1d_strided>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, offset: usize, stride: isize,
                len: usize) -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                check(unsafe {
                    ffi::rt_unary_1d_strided(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, offset as u64,
                        stride as i64, len as u64)
                })
            }

            fn [<apply_ $name _contiguous>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, start: usize, len: usize)
                -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                check(unsafe {
                    ffi::rt_unary_contiguous(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, start as u64, len as u64)
                })
            }
        }
    };
}

/// The four methods of one tensor-scalar op; `value` travels by address and is read before the call returns.
macro_rules! hip_scalar {
    ($name:ident, $code:expr $(, where $($bound:tt)+)?) => {
        paste! {
            fn [<scalar_apply_ $name>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, meta: &MetaTensor)
                -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                check(unsafe {
                    ffi::rt_scalar_nd(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, val(&value),
                        meta.offset as u64, meta.rank() as i32, meta.shape.as_slice().as_ptr() as *const u64,
                        meta.strides.as_slice().as_ptr() as *const i64)
                })
            }

            fn [<scalar_apply_ $name _nd>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, offset: usize,
                shape: &[usize], stride: &[isize]) -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                if shape.len() != stride.len() {
                    return Err(TensorError::WrongDims(format!("shape has {} dims, strides {}", shape.len(), stride.len())));
                }
                check(unsafe {
                    ffi::rt_scalar_nd(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, val(&value), offset as u64,
                        shape.len() as i32, shape.as_ptr() as *const u64, stride.as_ptr() as *const i64)
                })
            }

            fn [<scalar_apply_ $name _1d_strided>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T,
                offset: usize, stride: isize, len: usize) -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                check(unsafe {
                    ffi::rt_scalar_1d_strided(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, val(&value),
                        offset as u64, stride as i64, len as u64)
                })
            }

            fn [<scalar_apply_ $name _contiguous>]<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, start: usize,
                len: usize) -> Result<(), TensorError>
            $(where $($bound)+)?
            {
                check(unsafe {
                    ffi::rt_scalar_contiguous(self.raw(), dt::<T>(), $code, buf.ptr, buf.len as u64, val(&value),
                        start as u64, len as u64)
                })
            }
        }
    };
}

impl Backend for Hip {
    type Buf<T: TensorValue> = HipBuf<T>;

    fn device_type() -> DeviceType {
        DeviceType::Hip(0)
    }

    fn device(&self) -> DeviceType {
        DeviceType::Hip(self.ctx.device)
    }

    /// The trait gives `new` no way to fail.  A machine without a usable device gets a handle whose context is
    /// null; the library answers every call on a null context with RT_E_INVALID, so the failure surfaces as an
    /// `Err` from the first operation instead of a panic here.
    fn new() -> Self {
        Hip::construct(0).unwrap_or_else(|_| Hip { ctx: Arc::new(Ctx { raw: std::ptr::null_mut(), device: 0 }) })
    }

    fn alloc_from_slice<T: TensorValue>(&self, src: Box<[T]>) -> Result<Self::Buf<T>, TensorError> {
        let mut p = std::ptr::null_mut();
        check(unsafe { ffi::rt_alloc_from_slice(self.raw(), dt::<T>(), src.as_ptr() as *const c_void, src.len() as u64, &mut p) })?;
        Ok(self.wrap(p, src.len()))
    }

    /// Zero-filled, like `alloc_zeros` in backend/cuda.rs.
    fn alloc<T: TensorValue>(&self, len: usize) -> Result<Self::Buf<T>, TensorError> {
        let mut p = std::ptr::null_mut();
        check(unsafe { ffi::rt_alloc(self.raw(), dt::<T>(), len as u64, &mut p) })?;
        Ok(self.wrap(p, len))
    }

    fn copy_from_slice<T: TensorValue>(&self, dst: &mut Self::Buf<T>, src: &[T]) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_copy_from_slice(self.raw(), dt::<T>(), dst.ptr, dst.len as u64, src.as_ptr() as *const c_void,
                src.len() as u64)
        })
    }

    fn copy_range_within<T: TensorValue>(&self, dst: &mut Self::Buf<T>, src: &Self::Buf<T>, dst_offset: usize,
        src_offset: usize, len: usize) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_copy_range_within(self.raw(), dt::<T>(), dst.ptr, dst.len as u64, src.ptr, src.len as u64,
                dst_offset as u64, src_offset as u64, len as u64)
        })
    }

    fn read<T: TensorValue>(&self, buf: &Self::Buf<T>, offset: usize) -> Result<T, TensorError> {
        let mut out = std::mem::MaybeUninit::<T>::uninit();
        check(unsafe {
            ffi::rt_read(self.raw(), dt::<T>(), buf.ptr, buf.len as u64, offset as u64, out.as_mut_ptr() as *mut c_void)
        })?;
        Ok(unsafe { out.assume_init() })
    }

    fn write<T: TensorValue>(&self, buf: &mut Self::Buf<T>, offset: usize, value: T) -> Result<(), TensorError> {
        check(unsafe { ffi::rt_write(self.raw(), dt::<T>(), buf.ptr, buf.len as u64, offset as u64, val(&value)) })
    }

    fn len<T: TensorValue>(&self, buf: &Self::Buf<T>) -> usize {
        buf.len
    }

    fn copy<T: TensorValue>(&self, src: &Self::Buf<T>) -> Result<Self::Buf<T>, TensorError> {
        let mut p = std::ptr::null_mut();
        check(unsafe { ffi::rt_copy(self.raw(), dt::<T>(), src.ptr, src.len as u64, &mut p) })?;
        Ok(self.wrap(p, src.len))
    }

    fn dump<T: TensorValue>(&self, src: &Self::Buf<T>) -> Result<Box<[T]>, TensorError> {
        let mut host: Vec<T> = Vec::with_capacity(src.len);
        check(unsafe { ffi::rt_dump(self.raw(), dt::<T>(), src.ptr, src.len as u64, host.as_mut_ptr() as *mut c_void) })?;
        // rt_dump has written all `len` elements and waited for the copy
        unsafe { host.set_len(src.len) };
        Ok(host.into_boxed_slice())
    }

    /// All 13 x 13 dtype pairs on the device, with the semantics of Rust's `as` (core/value.rs:268-312).
    fn convert<T: TensorValue, N: TensorValue>(&self, src: &Self::Buf<T>, dst: &mut Self::Buf<N>) -> Result<(), TensorError> {
        check(unsafe { ffi::rt_convert(self.raw(), dt::<T>(), src.ptr, src.len as u64, dt::<N>(), dst.ptr, dst.len as u64) })
    }

    fn fill<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, meta: &MetaTensor) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fill_nd(self.raw(), dt::<T>(), buf.ptr, buf.len as u64, val(&value), meta.offset as u64,
                meta.rank() as i32, meta.shape.as_slice().as_ptr() as *const u64,
                meta.strides.as_slice().as_ptr() as *const i64)
        })
    }

    fn fill_nd<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, offset: usize, shape: &[usize], stride: &[isize])
        -> Result<(), TensorError> {
        if shape.len() != stride.len() {
            return Err(TensorError::WrongDims(format!("shape has {} dims, strides {}", shape.len(), stride.len())));
        }
        check(unsafe {
            ffi::rt_fill_nd(self.raw(), dt::<T>(), buf.ptr, buf.len as u64, val(&value), offset as u64,
                shape.len() as i32, shape.as_ptr() as *const u64, stride.as_ptr() as *const i64)
        })
    }

    fn fill_1d_strided<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, offset: usize, stride: isize, len: usize)
        -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fill_1d_strided(self.raw(), dt::<T>(), buf.ptr, buf.len as u64, val(&value), offset as u64,
                stride as i64, len as u64)
        })
    }

    fn fill_contiguous<T: TensorValue>(&self, buf: &mut Self::Buf<T>, value: T, start: usize, len: usize)
        -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fill_contiguous(self.raw(), dt::<T>(), buf.ptr, buf.len as u64, val(&value), start as u64, len as u64)
        })
    }

    /// `dst` may be the same buffer as `left` with the same layout (the in-place operators); the three metas share
    /// the broadcast shape and differ in strides, zero where an operand is expanded (ops/broadcast/mod.rs:20-60).
    fn broadcast<T: TensorValue>(&self, left: (*const Self::Buf<T>, &MetaTensor), right: (*const Self::Buf<T>, &MetaTensor),
        dst: (*mut Self::Buf<T>, &MetaTensor), op: BinaryOpType) -> Result<(), TensorError> {
        let (lbuf, lmeta) = left;
        let (rbuf, rmeta) = right;
        let (dbuf, dmeta) = dst;
        let rank = dmeta.rank();
        if lmeta.rank() != rank || rmeta.rank() != rank {
            return Err(TensorError::BroadcastError(format!(
                "operands of rank {} and {} against a destination of rank {rank}", lmeta.rank(), rmeta.rank())));
        }
        // raw pointers: `dst` and `left` may alias, so no `&mut` to one may exist beside a `&` to the other
        let (lp, ll) = unsafe { ((*lbuf).ptr, (*lbuf).len) };
        let (rp, rl) = unsafe { ((*rbuf).ptr, (*rbuf).len) };
        let (dp, dl) = unsafe { ((*dbuf).ptr, (*dbuf).len) };
        check(unsafe {
            ffi::rt_broadcast(self.raw(), dt::<T>(), op as i32, rank as i32, dmeta.shape.as_slice().as_ptr() as *const u64,
                lp, ll as u64, lmeta.offset as u64, lmeta.strides.as_slice().as_ptr() as *const i64,
                rp, rl as u64, rmeta.offset as u64, rmeta.strides.as_slice().as_ptr() as *const i64,
                dp, dl as u64, dmeta.offset as u64, dmeta.strides.as_slice().as_ptr() as *const i64)
        })
    }

    hip_unary! {neg, ffi::RT_U_NEG, where T: std::ops::Neg<Output = T>}
    hip_unary! {relu, ffi::RT_U_RELU}
    hip_unary! {sigmoid, ffi::RT_U_SIGMOID, where T: InvExp}
    hip_unary! {silu, ffi::RT_U_SILU, where T: InvExp}
    hip_unary! {tanh, ffi::RT_U_TANH, where T: Exp + InvExp}
    hip_unary! {abs, ffi::RT_U_ABS}
    hip_unary! {sqrt, ffi::RT_U_SQRT, where T: SquareRoot}
    hip_unary! {ln, ffi::RT_U_LN, where T: WeightValue}
    hip_unary! {expm1, ffi::RT_U_EXPM1, where T: Exp}
    hip_unary! {ln1p, ffi::RT_U_LN1P, where T: WeightValue}
    hip_unary! {floor, ffi::RT_U_FLOOR, where T: WeightValue}
    hip_unary! {ceil, ffi::RT_U_CEIL, where T: WeightValue}
    hip_unary! {round, ffi::RT_U_ROUND, where T: WeightValue}
    hip_unary! {trunc, ffi::RT_U_TRUNC, where T: WeightValue}

    hip_scalar! {add, ffi::RT_S_ADD}
    hip_scalar! {sub, ffi::RT_S_SUB}
    hip_scalar! {mul, ffi::RT_S_MUL}
    hip_scalar! {div, ffi::RT_S_DIV}
    hip_scalar! {log, ffi::RT_S_LOG, where T: WeightValue}
    hip_scalar! {log1p, ffi::RT_S_LOG1P, where T: WeightValue}
    hip_scalar! {leaky_relu, ffi::RT_S_LEAKY_RELU}
    hip_scalar! {elu, ffi::RT_S_ELU, where T: WeightValue}

    hip_unary! {sin, ffi::RT_U_SIN, where T: WeightValue}
    hip_unary! {cos, ffi::RT_U_COS, where T: WeightValue}
    hip_unary! {tan, ffi::RT_U_TAN, where T: WeightValue}
    hip_unary! {asin, ffi::RT_U_ASIN, where T: WeightValue}
    hip_unary! {acos, ffi::RT_U_ACOS, where T: WeightValue}
    hip_unary! {atan, ffi::RT_U_ATAN, where T: WeightValue}
    hip_unary! {sinh, ffi::RT_U_SINH, where T: WeightValue}
    hip_unary! {cosh, ffi::RT_U_COSH, where T: WeightValue}
    hip_unary! {asinh, ffi::RT_U_ASINH, where T: WeightValue}
    hip_unary! {acosh, ffi::RT_U_ACOSH, where T: WeightValue}
    hip_unary! {atanh, ffi::RT_U_ATANH, where T: WeightValue}
    hip_unary! {rsqrt, ffi::RT_U_RSQRT, where T: WeightValue}
    hip_unary! {reciprocal, ffi::RT_U_RECIPROCAL, where T: WeightValue}
    hip_unary! {square, ffi::RT_U_SQUARE, where T: WeightValue}
    hip_unary! {cube, ffi::RT_U_CUBE, where T: WeightValue}
    hip_unary! {exp, ffi::RT_U_EXP, where T: WeightValue}
    hip_unary! {sign, ffi::RT_U_SIGN, where T: WeightValue}

    fn apply_reduce_contiguous_flat<T: WeightValue>(&self, src: &Self::Buf<T>, dst: &mut Self::Buf<T>, start: usize,
        len: usize, op: ReductionOpTypes) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_reduce_flat(self.raw(), dt::<T>(), reduce_word(&op), src.ptr, src.len as u64, dst.ptr, dst.len as u64,
                start as u64, len as u64)
        })
    }

    fn apply_reduce_contiguous_nd<T: WeightValue>(&self, src: (&Self::Buf<T>, &MetaTensor), dst: (&mut Self::Buf<T>, &MetaTensor),
        dim: Dim, op: ReductionOpTypes) -> Result<(), TensorError> {
        let (sbuf, smeta) = src;
        let (dbuf, _) = dst; // the result is written densely from element 0, as backend/cuda.rs does
        check(unsafe {
            ffi::rt_reduce_nd(self.raw(), dt::<T>(), reduce_word(&op), sbuf.ptr, sbuf.len as u64, smeta.offset as u64,
                smeta.rank() as i32, smeta.shape.as_slice().as_ptr() as *const u64,
                smeta.strides.as_slice().as_ptr() as *const i64, dbuf.ptr, dbuf.len as u64, dim as i32)
        })
    }

    fn apply_argmax_contiguous_flat<T: WeightValue>(&self, src: &Self::Buf<T>, dst: &mut Self::Buf<u64>, start: usize,
        len: usize, op: ReductionOpTypes) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_argmax_flat(self.raw(), dt::<T>(), op.get_code() as i32, src.ptr, src.len as u64, dst.ptr as *mut u64,
                dst.len as u64, start as u64, len as u64)
        })
    }

    fn apply_argmax_contiguous_nd<T: WeightValue>(&self, src: (&Self::Buf<T>, &MetaTensor),
        dst: (&mut Self::Buf<u64>, &MetaTensor), dim: Dim, op: ReductionOpTypes) -> Result<(), TensorError> {
        let (sbuf, smeta) = src;
        let (dbuf, _) = dst;
        check(unsafe {
            ffi::rt_argmax_nd(self.raw(), dt::<T>(), op.get_code() as i32, sbuf.ptr, sbuf.len as u64, smeta.offset as u64,
                smeta.rank() as i32, smeta.shape.as_slice().as_ptr() as *const u64,
                smeta.strides.as_slice().as_ptr() as *const i64, dbuf.ptr as *mut u64, dbuf.len as u64, dim as i32)
        })
    }

    /// Convolution is outside this backend.  An `Err`, never `todo!()`: the remote server treats a backend panic
    /// as fatal (backend/remote/server.rs:112-114).
    fn apply_conv_2d<T: WeightValue>(&self, _input: (&Self::Buf<T>, &MetaTensor), _kernel: (&Self::Buf<T>, &MetaTensor),
        _output: &mut Self::Buf<T>, _config: &ConvConfig2D) -> Result<(), TensorError> {
        Err(TensorError::UnsupportedOperation("conv_2d is not implemented on the Hip backend".to_string()))
    }
}

/// One impl for every dtype: f32 / f64 reach rocBLAS inside the library, the others its tiled kernel
/// (the reference has one macro expansion per dtype, backend/cuda.rs:1517-1720).
impl<T: TensorValue> BackendMatMul<T> for Hip {
    fn matmul(&self, lhs: (&Self::Buf<T>, &MetaTensor, ContiguityTypes), rhs: (&Self::Buf<T>, &MetaTensor, ContiguityTypes),
        dst: &mut Self::Buf<T>, b: usize, m: usize, k: usize, n: usize) -> Result<(), TensorError> {
        let (lbuf, lmeta, lcont) = lhs;
        let (rbuf, rmeta, rcont) = rhs;
        check(unsafe {
            ffi::rt_matmul(self.raw(), dt::<T>(),
                lbuf.ptr, lbuf.len as u64, lmeta.offset as u64, lmeta.rank() as i32,
                lmeta.shape.as_slice().as_ptr() as *const u64, lmeta.strides.as_slice().as_ptr() as *const i64,
                contiguity_code(&lcont),
                rbuf.ptr, rbuf.len as u64, rmeta.offset as u64, rmeta.rank() as i32,
                rmeta.shape.as_slice().as_ptr() as *const u64, rmeta.strides.as_slice().as_ptr() as *const i64,
                contiguity_code(&rcont),
                dst.ptr, dst.len as u64, b as u64, m as u64, k as u64, n as u64)
        })
    }
}

/// The fused passes of `relu(x + bias)` under an L1 loss: the only entry points with no trait method behind them.
/// A caller that recognises the pattern on its tape (ops/unary/mod.rs:213-252 for ReLU, the L1 loss's sign map)
/// uses them instead of one launch per node; f32 and f64 only, anything else is RT_E_DTYPE -> `UnsupportedOperation`.
impl Hip {
    /// `y[r, c] = max(x[r, c] + bias[c], 0)` over a dense `rows x cols` matrix.
    pub fn fused_bias_relu<T: WeightValue>(&self, x: &HipBuf<T>, bias: &HipBuf<T>, y: &mut HipBuf<T>, rows: usize, cols: usize)
        -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fused_bias_relu(self.raw(), dt::<T>(), x.ptr, x.len as u64, bias.ptr, bias.len as u64, y.ptr,
                y.len as u64, rows as u64, cols as u64)
        })
    }

    /// `gmap = sign map of (y - target)`, `loss[0] = mean |y - target|` over `n` elements.
    pub fn fused_l1_forward<T: WeightValue>(&self, y: &HipBuf<T>, target: &HipBuf<T>, gmap: &mut HipBuf<T>,
        loss: &mut HipBuf<T>, n: usize) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fused_l1_forward(self.raw(), dt::<T>(), y.ptr, y.len as u64, target.ptr, target.len as u64, gmap.ptr,
                gmap.len as u64, loss.ptr, loss.len as u64, n as u64)
        })
    }

    /// `dbias[c] = sum over r of gmap[r, c] * upstream[0] / (rows * cols) * (y[r, c] > 0)`.
    pub fn fused_l1_relu_backward<T: WeightValue>(&self, gmap: &HipBuf<T>, y: &HipBuf<T>, upstream: &HipBuf<T>,
        dbias: &mut HipBuf<T>, rows: usize, cols: usize) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fused_l1_relu_backward(self.raw(), dt::<T>(), gmap.ptr, gmap.len as u64, y.ptr, y.len as u64,
                upstream.ptr, upstream.len as u64, dbias.ptr, dbias.len as u64, rows as u64, cols as u64)
        })
    }

    /// `y = relu(x + bias)` and `loss[0] = mean |y - target|` in one pass; with `fused_l1_relu_backward_t` the whole step
    /// without a stored gradient map.
    pub fn fused_bias_relu_l1<T: WeightValue>(&self, x: &HipBuf<T>, bias: &HipBuf<T>, target: &HipBuf<T>, y: &mut HipBuf<T>,
        loss: &mut HipBuf<T>, rows: usize, cols: usize) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fused_bias_relu_l1(self.raw(), dt::<T>(), x.ptr, x.len as u64, bias.ptr, bias.len as u64, target.ptr,
                target.len as u64, y.ptr, y.len as u64, loss.ptr, loss.len as u64, rows as u64, cols as u64)
        })
    }

    /// `dbias[c] = sum over r of (y[r, c] > 0) * ((sign(y[r, c] - target[r, c]) / (rows * cols)) * upstream[0])`.
    pub fn fused_l1_relu_backward_t<T: WeightValue>(&self, y: &HipBuf<T>, target: &HipBuf<T>, upstream: &HipBuf<T>,
        dbias: &mut HipBuf<T>, rows: usize, cols: usize) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_fused_l1_relu_backward_t(self.raw(), dt::<T>(), y.ptr, y.len as u64, target.ptr, target.len as u64,
                upstream.ptr, upstream.len as u64, dbias.ptr, dbias.len as u64, rows as u64, cols as u64)
        })
    }

    /// A program of up to `RT_CHAIN_MAX_STEPS` elementwise steps in one pass: `dst[dst_start + i] = steps(inputs[0][start0 + i])`,
    /// each input read once, the result written once.  The reference issues `relu(a * 3.0 + b) - 1.0` as four kernels and two
    /// clones (ops/scalar/add.rs:84-113, ops/unary/mod.rs:114-126); every step here is the same operation on `T` in the same
    /// order, so the result is bit for bit the same.  Build steps with `ChainStep::{unary, scalar, binary, binary_rev}`.
    /// `RT_E_DTYPE` (-> `UnsupportedOperation`) names a step that is not available in a chain: issue the separate ops then.
    pub fn fused_chain<T: TensorValue>(&self, inputs: &[(&HipBuf<T>, usize)], steps: &[ChainStep], len: usize,
        dst: &mut HipBuf<T>, dst_start: usize) -> Result<(), TensorError> {
        let ptrs: Vec<*const c_void> = inputs.iter().map(|(b, _)| b.ptr as *const c_void).collect();
        let lens: Vec<u64> = inputs.iter().map(|(b, _)| b.len as u64).collect();
        let starts: Vec<u64> = inputs.iter().map(|(_, s)| *s as u64).collect();
        let raw: Vec<ffi::rt_chain_step> = steps.iter().map(|s| s.0).collect();
        check(unsafe {
            ffi::rt_fused_chain(self.raw(), dt::<T>(), ptrs.len() as i32, ptrs.as_ptr(), lens.as_ptr(), starts.as_ptr(),
                len as u64, raw.len() as i32, raw.as_ptr(), dst.ptr, dst.len as u64, dst_start as u64)
        })
    }

    /// As `fused_chain`, in place on `inputs[which]`'s own run (the one aliasing the entry point allows).
    pub fn fused_chain_inplace<T: TensorValue>(&self, target: &mut HipBuf<T>, start: usize, others: &[(&HipBuf<T>, usize)],
        steps: &[ChainStep], len: usize) -> Result<(), TensorError> {
        let mut ptrs: Vec<*const c_void> = vec![target.ptr as *const c_void];
        let mut lens: Vec<u64> = vec![target.len as u64];
        let mut starts: Vec<u64> = vec![start as u64];
        for (b, s) in others {
            ptrs.push(b.ptr as *const c_void);
            lens.push(b.len as u64);
            starts.push(*s as u64);
        }
        let raw: Vec<ffi::rt_chain_step> = steps.iter().map(|s| s.0).collect();
        check(unsafe {
            ffi::rt_fused_chain(self.raw(), dt::<T>(), ptrs.len() as i32, ptrs.as_ptr(), lens.as_ptr(), starts.as_ptr(),
                len as u64, raw.len() as i32, raw.as_ptr(), target.ptr, target.len as u64, start as u64)
        })
    }

    /// One pass for a value-returning unary op on a contiguous operand (`alloc` + this, instead of `owned()` + the
    /// in-place op, which is two passes: ops/unary/mod.rs:114-126).
    pub fn unary_to<T: TensorValue>(&self, op: i32, src: &HipBuf<T>, start: usize, len: usize, dst: &mut HipBuf<T>)
        -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_unary_to(self.raw(), dt::<T>(), op, src.ptr, src.len as u64, start as u64, len as u64, dst.ptr,
                dst.len as u64)
        })
    }

    /// As `unary_to`, for a tensor-scalar op (ops/scalar/add.rs:93-97).
    pub fn scalar_to<T: TensorValue>(&self, op: i32, src: &HipBuf<T>, value: T, start: usize, len: usize,
        dst: &mut HipBuf<T>) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_scalar_to(self.raw(), dt::<T>(), op, src.ptr, src.len as u64, val(&value), start as u64, len as u64,
                dst.ptr, dst.len as u64)
        })
    }

    /// Dense row-major copy of a view in one launch (`view_to_contiguous`, core/tensor.rs:299-325, issues one
    /// `copy_range_within` per contiguous run).
    pub fn gather<T: TensorValue>(&self, src: &HipBuf<T>, meta: &MetaTensor, dst: &mut HipBuf<T>) -> Result<(), TensorError> {
        check(unsafe {
            ffi::rt_gather(self.raw(), dt::<T>(), src.ptr, src.len as u64, meta.offset as u64, meta.rank() as i32,
                meta.shape.as_slice().as_ptr() as *const u64, meta.strides.as_slice().as_ptr() as *const i64, dst.ptr,
                dst.len as u64)
        })
    }
}

/// One step of `Hip::fused_chain`.
#[derive(Clone, Copy, Debug)]
pub struct ChainStep(ffi::rt_chain_step);

impl ChainStep {
    /// `acc = op(acc)`, `op` one of `ffi::RT_U_*`.
    pub fn unary(op: i32) -> Self {
        ChainStep(ffi::rt_chain_step { kind: ffi::RT_CHAIN_UNARY, op, ..Default::default() })
    }
    /// `acc = acc op value`, `op` one of `ffi::RT_S_*`; the value travels in `T`'s own representation.
    pub fn scalar<T: TensorValue>(op: i32, value: T) -> Self {
        let mut raw = [0u8; 8];
        let n = std::mem::size_of::<T>().min(8);
        unsafe { std::ptr::copy_nonoverlapping(&value as *const T as *const u8, raw.as_mut_ptr(), n) };
        ChainStep(ffi::rt_chain_step { kind: ffi::RT_CHAIN_SCALAR, op, value: raw, ..Default::default() })
    }
    /// `acc = acc op inputs[operand]`, `op` a `BinaryOpType` code (ops/base.rs:7-12).
    pub fn binary(op: BinaryOpType, operand: usize) -> Self {
        ChainStep(ffi::rt_chain_step { kind: ffi::RT_CHAIN_BINARY, op: op as i32, operand: operand as i32, ..Default::default() })
    }
    /// `acc = inputs[operand] op acc`.
    pub fn binary_rev(op: BinaryOpType, operand: usize) -> Self {
        ChainStep(ffi::rt_chain_step { kind: ffi::RT_CHAIN_BINARY_REV, op: op as i32, operand: operand as i32, ..Default::default() })
    }
}

//! `HipBackend`: catgrad's interpreter `Backend` over libcatgrad_hip.so (MI355X / gfx950).
//!
//! Drop this file in as `catgrad/src/interpreter/backend/hip.rs`, add
//! `#[cfg(feature = "hip-backend")] pub mod hip;` next to the other backends in
//! `catgrad/src/interpreter/backend/mod.rs` (lines 10-14 there) and a `hip-backend`
//! feature in `catgrad/Cargo.toml`; link with `-lcatgrad_hip` (a `cargo:rustc-link-lib=dylib=catgrad_hip` line in build.rs).
//!
//! The shim is mechanical: every trait method forwards to the C entry point that
//! include/catgrad_hip.h declares for it.  The C ABI has the trait's own ownership model —
//! tensor arguments are consumed — so `HipTensor::into_raw` hands the reference over and
//! nothing is released twice.  A non-zero status becomes the panic the reference raises on
//! this path (the only `Result` is `ndarray_from_vec_*`'s `BackendError::ShapeError`).
//!
//! NOT COMPILED in the build container (it has no Rust toolchain); it is written against
//! `backend/mod.rs:24-132` and `interpreter/types.rs:28-34` and kept free of cleverness so
//! that it can be reviewed by eye.

use super::super::types::*;
use crate::category::core::{Dtype, Shape};
use crate::interpreter::backend::{Backend, BackendError, BackendTensorOps};
use std::ffi::{c_char, c_int, c_uint, c_void, CStr};
use std::sync::Arc;

#[repr(C)]
pub struct CgBackend {
    _private: [u8; 0],
}
#[repr(C)]
pub struct CgTensor {
    _private: [u8; 0],
}

const CG_F32: c_int = 0;
const CG_F16: c_int = 1;
const CG_BF16: c_int = 2;
const CG_F8: c_int = 3;
const CG_U32: c_int = 4;
const CG_ERR_SHAPE: c_int = 1;

#[link(name = "catgrad_hip")]
extern "C" {
    fn cg_backend_create(device: c_int, out: *mut *mut CgBackend) -> c_int;
    fn cg_backend_destroy(b: *mut CgBackend);
    fn cg_last_error() -> *const c_char;
    fn cg_tensor_retain(t: *mut CgTensor);
    fn cg_tensor_release(t: *mut CgTensor);
    fn cg_tensor_rank(t: *const CgTensor) -> usize;
    fn cg_tensor_shape(t: *const CgTensor, dims: *mut usize);
    fn cg_tensor_numel(t: *const CgTensor) -> usize;
    fn cg_zeros(b: *mut CgBackend, dt: c_int, dims: *const usize, rank: usize, out: *mut *mut CgTensor) -> c_int;
    fn cg_from_host(b: *mut CgBackend, dt: c_int, data: *const c_void, len: usize, dims: *const usize, rank: usize,
                    out: *mut *mut CgTensor) -> c_int;
    fn cg_arange(b: *mut CgBackend, end: usize, out: *mut *mut CgTensor) -> c_int;
    fn cg_to_host(b: *mut CgBackend, t: *const CgTensor, dst: *mut c_void, len: usize) -> c_int;
    fn cg_to_bool(b: *mut CgBackend, t: *const CgTensor, out: *mut c_int) -> c_int;
    fn cg_compare(b: *mut CgBackend, x: *const CgTensor, y: *const CgTensor, out: *mut c_int) -> c_int;
    fn cg_format_tensor(b: *mut CgBackend, t: *const CgTensor, buf: *mut c_char, cap: usize) -> c_int;
    fn cg_cast(b: *mut CgBackend, x: *mut CgTensor, dt: c_int, out: *mut *mut CgTensor) -> c_int;
    fn cg_unary(b: *mut CgBackend, op: c_uint, x: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
    fn cg_binary(b: *mut CgBackend, op: c_uint, x: *mut CgTensor, y: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
    fn cg_where(b: *mut CgBackend, m: *mut CgTensor, x: *mut CgTensor, y: *mut CgTensor, out: *mut *mut CgTensor)
                -> c_int;
    fn cg_matmul(b: *mut CgBackend, x: *mut CgTensor, y: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
    fn cg_sum(b: *mut CgBackend, x: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
    fn cg_max(b: *mut CgBackend, x: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
    fn cg_argmax(b: *mut CgBackend, x: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
    fn cg_topk(b: *mut CgBackend, x: *mut CgTensor, k: usize, values: *mut *mut CgTensor, indices: *mut *mut CgTensor)
               -> c_int;
    fn cg_broadcast(b: *mut CgBackend, x: *mut CgTensor, dims: *const usize, rank: usize, out: *mut *mut CgTensor)
                    -> c_int;
    fn cg_reshape(b: *mut CgBackend, x: *mut CgTensor, dims: *const usize, rank: usize, out: *mut *mut CgTensor)
                  -> c_int;
    fn cg_transpose(b: *mut CgBackend, x: *mut CgTensor, d0: usize, d1: usize, out: *mut *mut CgTensor) -> c_int;
    fn cg_slice(b: *mut CgBackend, x: *mut CgTensor, dim: usize, start: usize, len: usize, out: *mut *mut CgTensor)
                -> c_int;
    fn cg_concat(b: *mut CgBackend, x: *mut CgTensor, y: *mut CgTensor, dim: usize, out: *mut *mut CgTensor) -> c_int;
    fn cg_index(b: *mut CgBackend, x: *mut CgTensor, dim: usize, idx: *mut CgTensor, out: *mut *mut CgTensor) -> c_int;
}

// cg_unary_op / cg_binary_op, in header order.
#[rustfmt::skip]
mod op {
    pub const NEG: u32 = 0; pub const SIN: u32 = 1; pub const COS: u32 = 2; pub const EXP: u32 = 3;
    pub const LOG: u32 = 4; pub const FLOOR: u32 = 5; pub const ROUND: u32 = 6;
    pub const ADD: u32 = 0; pub const SUB: u32 = 1; pub const MUL: u32 = 2; pub const DIV: u32 = 3;
    pub const POW: u32 = 4; pub const LT: u32 = 5; pub const GT: u32 = 6; pub const GTE: u32 = 7;
    pub const LTE: u32 = 8; pub const EQ: u32 = 9;
}

fn last_error() -> String {
    unsafe { CStr::from_ptr(cg_last_error()).to_string_lossy().into_owned() }
}

/// Non-zero status => the panic the reference raises (e.g. "Shape mismatch in operation").
fn check(status: c_int) {
    if status != 0 {
        panic!("{}", last_error());
    }
}

struct Device(*mut CgBackend);
unsafe impl Send for Device {}
unsafe impl Sync for Device {}
impl Drop for Device {
    fn drop(&mut self) {
        unsafe { cg_backend_destroy(self.0) }
    }
}

/// One GPU, one stream, one memory pool.  `Clone` shares the same device context.
#[derive(Clone)]
pub struct HipBackend {
    device: Arc<Device>,
}

impl std::fmt::Debug for HipBackend {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HipBackend")
    }
}

impl HipBackend {
    pub fn new(device: i32) -> Self {
        let mut raw = std::ptr::null_mut();
        check(unsafe { cg_backend_create(device, &mut raw) });
        Self { device: Arc::new(Device(raw)) }
    }
    fn raw(&self) -> *mut CgBackend {
        self.device.0
    }
}

/// A reference-counted handle to a strided device view.  `Clone` is a refcount bump.
/// A tensor may outlive every `HipBackend` value (a `Parameters<HipBackend>` map dropped after the backend, a result
/// kept by the caller): the C library counts the live handles of a backend and `cg_backend_destroy` only gives up the
/// owner's hold, so `Drop` and `Clone` here stay valid in any drop order, as for the reference's tensors
/// (`BackendTensorOps`, mod.rs:124-126, has no lifetime tied to a backend).
pub struct HipTensor(*mut CgTensor);
unsafe impl Send for HipTensor {}
unsafe impl Sync for HipTensor {}

impl HipTensor {
    /// Gives this reference to a consuming C call.
    fn into_raw(self) -> *mut CgTensor {
        let p = self.0;
        std::mem::forget(self);
        p
    }
}
impl Clone for HipTensor {
    fn clone(&self) -> Self {
        unsafe { cg_tensor_retain(self.0) };
        HipTensor(self.0)
    }
}
impl Drop for HipTensor {
    fn drop(&mut self) {
        unsafe { cg_tensor_release(self.0) }
    }
}
impl std::fmt::Debug for HipTensor {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "HipTensor{:?}", self.shape().0)
    }
}
impl BackendTensorOps for HipTensor {
    fn shape(&self) -> Shape {
        let rank = unsafe { cg_tensor_rank(self.0) };
        let mut dims = vec![0usize; rank];
        unsafe { cg_tensor_shape(self.0, dims.as_mut_ptr()) };
        Shape(dims)
    }
}

fn dtype_code(d: &Dtype) -> c_int {
    match d {
        Dtype::F32 => CG_F32,
        Dtype::F16 => CG_F16,
        Dtype::BF16 => CG_BF16,
        Dtype::F8 => CG_F8,
        Dtype::U32 => CG_U32,
    }
}

fn dtype_of<const N: usize>(x: &TaggedTensorTuple<HipBackend, N>) -> Dtype {
    match x {
        TaggedTensorTuple::F32(_) => Dtype::F32,
        TaggedTensorTuple::F16(_) => Dtype::F16,
        TaggedTensorTuple::BF16(_) => Dtype::BF16,
        TaggedTensorTuple::FP8(_) => Dtype::F8,
        TaggedTensorTuple::U32(_) => Dtype::U32,
    }
}

fn tag_for(dtype: &Dtype, t: HipTensor) -> TaggedTensor<HipBackend> {
    match dtype {
        Dtype::F32 => TaggedTensor::F32([t]),
        Dtype::F16 => TaggedTensor::F16([t]),
        Dtype::BF16 => TaggedTensor::BF16([t]),
        Dtype::F8 => TaggedTensor::FP8([t]),
        Dtype::U32 => TaggedTensor::U32([t]),
    }
}

fn untag<const N: usize>(x: TaggedTensorTuple<HipBackend, N>) -> [HipTensor; N] {
    match x {
        TaggedTensorTuple::F32(a)
        | TaggedTensorTuple::F16(a)
        | TaggedTensorTuple::BF16(a)
        | TaggedTensorTuple::FP8(a)
        | TaggedTensorTuple::U32(a) => a,
    }
}

impl HipBackend {
    fn unary(&self, code: u32, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        let dt = x.dtype();
        let [t] = untag(x);
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_unary(self.raw(), code, t.into_raw(), &mut out) });
        tag_for(&dt, HipTensor(out))
    }
    fn binary(&self, code: u32, x: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        let dt = dtype_of(&x);
        let [a, b] = untag(x);
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_binary(self.raw(), code, a.into_raw(), b.into_raw(), &mut out) });
        tag_for(&dt, HipTensor(out))
    }
    fn one(&self, x: TaggedTensor<Self>, out_dtype: Option<Dtype>,
           f: impl FnOnce(*mut CgBackend, *mut CgTensor, *mut *mut CgTensor) -> c_int) -> TaggedTensor<Self> {
        let dt = out_dtype.unwrap_or_else(|| x.dtype());
        let [t] = untag(x);
        let mut out = std::ptr::null_mut();
        check(f(self.raw(), t.into_raw(), &mut out));
        tag_for(&dt, HipTensor(out))
    }
    fn from_host(&self, dt: Dtype, data: *const c_void, len: usize, shape: Shape)
                 -> Result<TaggedTensor<Self>, BackendError> {
        let mut out = std::ptr::null_mut();
        let st = unsafe { cg_from_host(self.raw(), dtype_code(&dt), data, len, shape.0.as_ptr(), shape.0.len(), &mut out) };
        if st == CG_ERR_SHAPE {
            return Err(BackendError::ShapeError);
        }
        check(st);
        Ok(tag_for(&dt, HipTensor(out)))
    }
}

impl Backend for HipBackend {
    type BackendTensor = HipTensor;

    fn zeros(&self, shape: Shape, target_dtype: Dtype) -> TaggedTensor<Self> {
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_zeros(self.raw(), dtype_code(&target_dtype), shape.0.as_ptr(), shape.0.len(), &mut out) });
        tag_for(&target_dtype, HipTensor(out))
    }

    fn ndarray_from_vec_f32(&self, data: Vec<f32>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        self.from_host(Dtype::F32, data.as_ptr() as *const c_void, data.len(), shape)
    }
    fn ndarray_from_vec_f16(&self, data: Vec<half::f16>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        self.from_host(Dtype::F16, data.as_ptr() as *const c_void, data.len(), shape)
    }
    fn ndarray_from_vec_bf16(&self, data: Vec<half::bf16>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        self.from_host(Dtype::BF16, data.as_ptr() as *const c_void, data.len(), shape)
    }
    fn ndarray_from_vec_fp8(&self, data: Vec<float8::F8E4M3>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        self.from_host(Dtype::F8, data.as_ptr() as *const c_void, data.len(), shape)
    }
    fn ndarray_from_vec_u32(&self, data: Vec<u32>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        self.from_host(Dtype::U32, data.as_ptr() as *const c_void, data.len(), shape)
    }

    fn cast(&self, x: TaggedTensor<Self>, target_dtype: Dtype) -> TaggedTensor<Self> {
        let code = dtype_code(&target_dtype);
        self.one(x, Some(target_dtype), |b, t, o| unsafe { cg_cast(b, t, code, o) })
    }
    fn matmul(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        let dt = dtype_of(&lhs);
        let [a, b] = untag(lhs);
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_matmul(self.raw(), a.into_raw(), b.into_raw(), &mut out) });
        tag_for(&dt, HipTensor(out))
    }
    fn add(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::ADD, lhs) }
    fn sub(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::SUB, lhs) }
    fn mul(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::MUL, lhs) }
    fn div(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::DIV, lhs) }
    fn pow(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::POW, lhs) }
    fn lt(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::LT, lhs) }
    fn gt(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::GT, lhs) }
    fn gte(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::GTE, lhs) }
    fn lte(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::LTE, lhs) }
    fn eq(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> { self.binary(op::EQ, lhs) }

    fn where_cond(&self, args: TaggedTensorTuple<Self, 3>) -> TaggedTensor<Self> {
        let dt = dtype_of(&args);
        let [m, x, y] = untag(args);
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_where(self.raw(), m.into_raw(), x.into_raw(), y.into_raw(), &mut out) });
        tag_for(&dt, HipTensor(out))
    }

    fn sin(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::SIN, x) }
    fn cos(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::COS, x) }
    fn exp(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::EXP, x) }
    fn log(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::LOG, x) }
    fn floor(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::FLOOR, x) }
    fn round(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::ROUND, x) }
    fn neg(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> { self.unary(op::NEG, x) }

    fn broadcast(&self, x: TaggedTensor<Self>, shape: Shape) -> TaggedTensor<Self> {
        self.one(x, None, |b, t, o| unsafe { cg_broadcast(b, t, shape.0.as_ptr(), shape.0.len(), o) })
    }
    fn reshape(&self, x: TaggedTensor<Self>, new_shape: Shape) -> TaggedTensor<Self> {
        self.one(x, None, |b, t, o| unsafe { cg_reshape(b, t, new_shape.0.as_ptr(), new_shape.0.len(), o) })
    }
    fn transpose(&self, x: TaggedTensor<Self>, dim0: usize, dim1: usize) -> TaggedTensor<Self> {
        self.one(x, None, |b, t, o| unsafe { cg_transpose(b, t, dim0, dim1, o) })
    }
    fn max(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.one(x, None, |b, t, o| unsafe { cg_max(b, t, o) })
    }
    fn sum(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.one(x, None, |b, t, o| unsafe { cg_sum(b, t, o) })
    }
    fn argmax(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.one(x, Some(Dtype::U32), |b, t, o| unsafe { cg_argmax(b, t, o) })
    }
    fn topk(&self, x: TaggedTensor<Self>, k: usize) -> (TaggedTensor<Self>, TaggedTensor<Self>) {
        let dt = x.dtype(); // the values keep the input's dtype (cg_topk takes every floating-point dtype)
        let [t] = untag(x);
        let (mut v, mut i) = (std::ptr::null_mut(), std::ptr::null_mut());
        check(unsafe { cg_topk(self.raw(), t.into_raw(), k, &mut v, &mut i) });
        (tag_for(&dt, HipTensor(v)), TaggedTensor::U32([HipTensor(i)]))
    }
    fn compare(&self, x: TaggedTensorTuple<Self, 2>) -> bool {
        let [a, b] = untag(x);
        let mut r: c_int = 0;
        check(unsafe { cg_compare(self.raw(), a.0, b.0, &mut r) }); // borrowing call; a, b drop afterwards
        r != 0
    }
    fn concat(&self, x: TaggedTensor<Self>, y: TaggedTensor<Self>, dim: usize) -> TaggedTensor<Self> {
        if x.dtype() != y.dtype() {
            panic!("Incompatible types for concatenation");
        }
        let dt = x.dtype();
        let ([a], [b]) = (untag(x), untag(y));
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_concat(self.raw(), a.into_raw(), b.into_raw(), dim, &mut out) });
        tag_for(&dt, HipTensor(out))
    }
    fn index(&self, x: TaggedTensor<Self>, dim: usize, indices: TaggedTensor<Self>) -> TaggedTensor<Self> {
        if indices.dtype() != Dtype::U32 {
            panic!("Invalid input types for indexing");
        }
        let dt = x.dtype();
        let ([t], [ix]) = (untag(x), untag(indices));
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_index(self.raw(), t.into_raw(), dim, ix.into_raw(), &mut out) });
        tag_for(&dt, HipTensor(out))
    }
    fn slice(&self, x: TaggedTensor<Self>, dim: usize, start: usize, len: usize) -> TaggedTensor<Self> {
        self.one(x, None, |b, t, o| unsafe { cg_slice(b, t, dim, start, len, o) })
    }
    fn arange(&self, end: usize) -> TaggedTensor<Self> {
        let mut out = std::ptr::null_mut();
        check(unsafe { cg_arange(self.raw(), end, &mut out) });
        TaggedTensor::U32([HipTensor(out)])
    }

    fn to_bool(&self, x: TaggedTensor<Self>) -> bool {
        let [t] = untag(x);
        let mut r: c_int = 0;
        check(unsafe { cg_to_bool(self.raw(), t.0, &mut r) });
        r != 0
    }

    fn to_vec(&self, vec: TaggedTensor<Self>) -> TaggedVec {
        let dt = vec.dtype();
        let [t] = untag(vec);
        let n = unsafe { cg_tensor_numel(t.0) };
        match dt {
            Dtype::F32 => {
                let mut v = vec![0f32; n];
                check(unsafe { cg_to_host(self.raw(), t.0, v.as_mut_ptr() as *mut c_void, n) });
                TaggedVec::F32(v)
            }
            Dtype::U32 => {
                let mut v = vec![0u32; n];
                check(unsafe { cg_to_host(self.raw(), t.0, v.as_mut_ptr() as *mut c_void, n) });
                TaggedVec::U32(v)
            }
            Dtype::F16 => {
                // 2-byte elements: half::f16 is repr(transparent) over its u16 bit pattern
                let mut v = vec![half::f16::ZERO; n];
                check(unsafe { cg_to_host(self.raw(), t.0, v.as_mut_ptr() as *mut c_void, n) });
                TaggedVec::F16(v)
            }
            Dtype::BF16 => {
                let mut v = vec![half::bf16::ZERO; n];
                check(unsafe { cg_to_host(self.raw(), t.0, v.as_mut_ptr() as *mut c_void, n) });
                TaggedVec::BF16(v)
            }
            Dtype::F8 => {
                // 1-byte elements: float8::F8E4M3 is repr(transparent) over its u8 bit pattern
                let mut v = vec![float8::F8E4M3::ZERO; n];
                check(unsafe { cg_to_host(self.raw(), t.0, v.as_mut_ptr() as *mut c_void, n) });
                TaggedVec::FP8(v)
            }
        }
    }

    fn format_tensor(&self, tensor: &TaggedTensor<Self>) -> String {
        let t = match tensor {
            TaggedTensor::F32([t]) | TaggedTensor::F16([t]) | TaggedTensor::BF16([t]) | TaggedTensor::FP8([t])
            | TaggedTensor::U32([t]) => t,
        };
        let mut buf = vec![0 as c_char; 4096];
        check(unsafe { cg_format_tensor(self.raw(), t.0, buf.as_mut_ptr(), buf.len()) });
        unsafe { CStr::from_ptr(buf.as_ptr()).to_string_lossy().into_owned() }
    }
}

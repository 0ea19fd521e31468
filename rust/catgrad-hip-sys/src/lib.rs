//! `extern "C"` declarations of include/catgrad_hip.h: one function per method of catgrad's
//! `trait Backend` (catgrad/src/interpreter/backend/mod.rs:22-82) plus handle management.
//!
//! Conventions of the library: every function returns a status (0 = ok); tensor arguments are
//! borrowed; every `out` receives a new reference the caller releases with `cg_tensor_release`.
#![allow(non_camel_case_types)]
use std::os::raw::{c_char, c_int};

#[repr(C)]
pub struct cg_backend {
    _private: [u8; 0],
}
#[repr(C)]
pub struct cg_tensor {
    _private: [u8; 0],
}
#[repr(C)]
pub struct cg_params {
    _private: [u8; 0],
}

/// core::Dtype (catgrad/src/category/core.rs:20-24)
pub const CG_F32: c_int = 0;
pub const CG_U32: c_int = 1;

pub const CG_OK: c_int = 0;
/// BackendError::ShapeError and every "Shape mismatch" panic
pub const CG_ERR_SHAPE: c_int = 1;

/// cg_backend_create flags
pub const CG_FLAG_BF16: u32 = 1;
pub const CG_FLAG_EAGER: u32 = 2;
pub const CG_FLAG_NO_PATTERNS: u32 = 4;
pub const CG_FLAG_ATTN_ONE_PASS: u32 = 8;

pub type cg_out = *mut *mut cg_tensor;

extern "C" {
    // ---- backend lifetime
    pub fn cg_backend_create(device: c_int, flags: u32, out: *mut *mut cg_backend) -> c_int;
    pub fn cg_backend_destroy(be: *mut cg_backend);
    pub fn cg_last_error(be: *const cg_backend) -> *const c_char;
    pub fn cg_sync(be: *mut cg_backend) -> c_int;
    pub fn cg_tensor_realize(be: *mut cg_backend, t: *mut cg_tensor) -> c_int;
    pub fn cg_tensor_prefetch(be: *mut cg_backend, t: *mut cg_tensor) -> c_int;
    pub fn cg_backend_name(be: *const cg_backend) -> *const c_char;

    // ---- handles: Clone / Drop / BackendTensorOps::shape
    pub fn cg_tensor_retain(t: *mut cg_tensor) -> *mut cg_tensor;
    pub fn cg_tensor_release(t: *mut cg_tensor);
    pub fn cg_tensor_rank(t: *const cg_tensor) -> c_int;
    pub fn cg_tensor_shape(t: *const cg_tensor, dims: *mut usize) -> c_int;
    pub fn cg_tensor_dtype(t: *const cg_tensor) -> c_int;
    pub fn cg_tensor_size(t: *const cg_tensor) -> usize;

    // ---- Backend methods
    pub fn cg_zeros(be: *mut cg_backend, dims: *const usize, rank: c_int, dtype: c_int, out: cg_out) -> c_int;
    pub fn cg_from_f32(be: *mut cg_backend, data: *const f32, n: usize, dims: *const usize, rank: c_int, out: cg_out) -> c_int;
    pub fn cg_from_u32(be: *mut cg_backend, data: *const u32, n: usize, dims: *const usize, rank: c_int, out: cg_out) -> c_int;
    pub fn cg_from_bf16(be: *mut cg_backend, bits: *const u16, n: usize, dims: *const usize, rank: c_int, out: cg_out) -> c_int;
    pub fn cg_stack(be: *mut cg_backend, parts: *const *mut cg_tensor, n: usize, out: cg_out) -> c_int;
    pub fn cg_cast(be: *mut cg_backend, x: *mut cg_tensor, target: c_int, out: cg_out) -> c_int;
    pub fn cg_matmul(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_add(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_sub(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_mul(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_div(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_pow(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_lt(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_eq(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_sin(be: *mut cg_backend, x: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_cos(be: *mut cg_backend, x: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_neg(be: *mut cg_backend, x: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_broadcast(be: *mut cg_backend, x: *mut cg_tensor, dims: *const usize, rank: c_int, out: cg_out) -> c_int;
    pub fn cg_reshape(be: *mut cg_backend, x: *mut cg_tensor, dims: *const usize, rank: c_int, out: cg_out) -> c_int;
    pub fn cg_transpose(be: *mut cg_backend, x: *mut cg_tensor, dim0: usize, dim1: usize, out: cg_out) -> c_int;
    pub fn cg_max(be: *mut cg_backend, x: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_sum(be: *mut cg_backend, x: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_argmax(be: *mut cg_backend, x: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_argmax_into(be: *mut cg_backend, x: *mut cg_tensor, out: *mut cg_tensor) -> c_int;
    pub fn cg_topk(be: *mut cg_backend, x: *mut cg_tensor, k: usize, values: cg_out, indices: cg_out) -> c_int;
    pub fn cg_compare(be: *mut cg_backend, a: *mut cg_tensor, b: *mut cg_tensor, equal: *mut c_int) -> c_int;
    pub fn cg_concat(be: *mut cg_backend, x: *mut cg_tensor, y: *mut cg_tensor, dim: usize, out: cg_out) -> c_int;
    pub fn cg_index(be: *mut cg_backend, x: *mut cg_tensor, dim: usize, indices: *mut cg_tensor, out: cg_out) -> c_int;
    pub fn cg_slice(be: *mut cg_backend, x: *mut cg_tensor, dim: usize, start: usize, len: usize, out: cg_out) -> c_int;
    pub fn cg_arange(be: *mut cg_backend, end: usize, out: cg_out) -> c_int;
    pub fn cg_to_f32(be: *mut cg_backend, x: *mut cg_tensor, dst: *mut f32, n: usize) -> c_int;
    pub fn cg_to_u32(be: *mut cg_backend, x: *mut cg_tensor, dst: *mut u32, n: usize) -> c_int;

    // ---- weight files (catgrad-llm/examples/llama/main.rs:171-350)
    pub fn cg_params_create(out: *mut *mut cg_params) -> c_int;
    pub fn cg_params_destroy(p: *mut cg_params);
    pub fn cg_params_len(p: *const cg_params) -> usize;
    pub fn cg_params_key(p: *const cg_params, i: usize) -> *const c_char;
    pub fn cg_params_get(p: *const cg_params, path: *const c_char, out: cg_out) -> c_int;
    pub fn cg_params_load(be: *mut cg_backend, params: *mut cg_params, file: *const c_char, prefix: *const c_char, n_loaded: *mut usize) -> c_int;
    pub fn cg_params_stack_experts(be: *mut cg_backend, params: *mut cg_params, prefix: *const c_char, num_layers: usize, num_experts: usize) -> c_int;
    pub fn cg_weights_last_error() -> *const c_char;
}

//! MI355X (gfx950) backend: `impl Backend for HipBackend` over the C ABI of libcatgrad_hip.so.
//!
//! Every trait method forwards to the C function of the same name.  The trait takes its tensor
//! arguments by value; the C ABI borrows them, so the Rust wrappers are dropped after the call,
//! which gives the library the reference counts it uses to decide what may be fused, computed in
//! place or appended to (a KV cache moved into `Interpreter::run`).  Where the reference panics
//! (shape mismatch, sin of a U32 tensor, ...) the C function returns a status and this shim panics
//! with the library's message; the two constructors return `Err(BackendError::ShapeError)`.
use super::super::types::*;
use crate::category::core::{Dtype, Shape};
use crate::interpreter::backend::{Backend, BackendError, BackendTensorOps};
use catgrad_hip_sys as sys;
use std::ffi::CStr;
use std::fmt;
use std::ptr;
use std::sync::{Arc, Mutex};
use std::thread::{self, ThreadId};

// The library is single-threaded per backend: recording a graph, releasing a tensor and every other
// call edit unlocked per-backend state.  The trait's bounds still make the handles `Send + Sync`, so
// the rule is enforced here instead of being left to the caller: a backend is used on the thread that
// made it (`raw` panics elsewhere), a tensor dropped on another thread is parked in `GRAVEYARD` and
// released by its owner's next call, and the only thing other threads really do - `clone` and
// `shape` - is an atomic increment and a read of fields that never change.
struct Handle {
    be: *mut sys::cg_backend,
    owner: ThreadId,
}
unsafe impl Send for Handle {}
unsafe impl Sync for Handle {}
impl Drop for Handle {
    fn drop(&mut self) {
        // (the library keeps the backend alive until its last tensor is released)
        unsafe { sys::cg_backend_destroy(self.be) }
    }
}

/// tensors dropped away from their owner thread: (owner, pointer)
static GRAVEYARD: Mutex<Vec<(ThreadId, usize)>> = Mutex::new(Vec::new());

fn bury_or_release(owner: ThreadId, t: *mut sys::cg_tensor) {
    if thread::current().id() == owner {
        unsafe { sys::cg_tensor_release(t) }
    } else {
        GRAVEYARD.lock().unwrap().push((owner, t as usize));
    }
}

fn release_buried(owner: ThreadId) {
    let mine: Vec<usize> = {
        let mut g = GRAVEYARD.lock().unwrap();
        if g.is_empty() {
            return;
        }
        let (mine, rest): (Vec<_>, Vec<_>) = g.drain(..).partition(|(o, _)| *o == owner);
        *g = rest;
        mine.into_iter().map(|(_, p)| p).collect()
    };
    for p in mine {
        unsafe { sys::cg_tensor_release(p as *mut sys::cg_tensor) }
    }
}

/// One device, one stream.  `Clone` shares the handle.
#[derive(Clone)]
pub struct HipBackend(Arc<Handle>);

impl fmt::Debug for HipBackend {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        let name = unsafe { CStr::from_ptr(sys::cg_backend_name(self.raw())) };
        write!(f, "HipBackend({})", name.to_string_lossy())
    }
}

/// `BackendTensor`: an owned reference.  `Clone` = retain (O(1), an atomic increment), `Drop` =
/// release on the owner thread (parked for it otherwise).
pub struct HipTensor(*mut sys::cg_tensor, ThreadId);
unsafe impl Send for HipTensor {}
unsafe impl Sync for HipTensor {}
impl Clone for HipTensor {
    fn clone(&self) -> Self {
        HipTensor(unsafe { sys::cg_tensor_retain(self.0) }, self.1)
    }
}
impl Drop for HipTensor {
    fn drop(&mut self) {
        bury_or_release(self.1, self.0)
    }
}
impl fmt::Debug for HipTensor {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        write!(f, "HipTensor({:?})", self.shape().0)
    }
}
impl BackendTensorOps for HipTensor {
    /// host only: never waits for the device
    fn shape(&self) -> Shape {
        let rank = unsafe { sys::cg_tensor_rank(self.0) } as usize;
        let mut dims = vec![0usize; rank];
        unsafe { sys::cg_tensor_shape(self.0, dims.as_mut_ptr()) };
        Shape(dims)
    }
}

type Unary = unsafe extern "C" fn(*mut sys::cg_backend, *mut sys::cg_tensor, sys::cg_out) -> i32;
type Binary = unsafe extern "C" fn(*mut sys::cg_backend, *mut sys::cg_tensor, *mut sys::cg_tensor, sys::cg_out) -> i32;

fn dtype_code(d: Dtype) -> i32 {
    match d {
        Dtype::F32 => sys::CG_F32,
        Dtype::U32 => sys::CG_U32,
    }
}

impl HipBackend {
    /// `bf16`: weights handed over as F32 of rank >= 2 are stored as bf16 and matmuls round their
    /// operands to bf16 (f32 accumulation); everything else stays f32.
    pub fn new(device: i32, bf16: bool) -> Self {
        let mut be = ptr::null_mut();
        let flags = if bf16 { sys::CG_FLAG_BF16 } else { 0 };
        let st = unsafe { sys::cg_backend_create(device, flags, &mut be) };
        assert_eq!(st, sys::CG_OK, "cg_backend_create: no usable gfx950 device");
        HipBackend(Arc::new(Handle { be, owner: thread::current().id() }))
    }

    /// the backend pointer for a call into the library: only on the thread that made the backend
    fn raw(&self) -> *mut sys::cg_backend {
        assert_eq!(thread::current().id(), self.0.owner, "HipBackend is used on the thread that created it");
        release_buried(self.0.owner);
        self.0.be
    }

    /// the reference panics where the C ABI returns a status
    fn check(&self, st: i32) {
        if st != sys::CG_OK {
            let msg = unsafe { CStr::from_ptr(sys::cg_last_error(self.raw())) };
            panic!("{}", msg.to_string_lossy());
        }
    }

    /// (is F32, the tensor) of a tagged tensor
    fn untag(x: TaggedTensor<Self>) -> (bool, HipTensor) {
        match x {
            TaggedTensorTuple::F32([t]) => (true, t),
            TaggedTensorTuple::U32([t]) => (false, t),
        }
    }

    fn tag(f32_tag: bool, out: *mut sys::cg_tensor) -> TaggedTensor<Self> {
        if f32_tag {
            TaggedTensorTuple::F32([HipTensor(out, thread::current().id())])
        } else {
            TaggedTensorTuple::U32([HipTensor(out, thread::current().id())])
        }
    }

    /// a unary op whose result keeps the tag of its argument
    fn unary(&self, f: Unary, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        let (is_f32, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { f(self.raw(), t.0, &mut out) });
        Self::tag(is_f32, out)
    }

    /// a binary op whose result keeps the tag of its arguments (lt / eq too: ndarray.rs:164-198)
    fn binary(&self, f: Binary, args: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        let (is_f32, [a, b]) = match args {
            TaggedTensorTuple::F32(x) => (true, x),
            TaggedTensorTuple::U32(x) => (false, x),
        };
        let mut out = ptr::null_mut();
        self.check(unsafe { f(self.raw(), a.0, b.0, &mut out) });
        Self::tag(is_f32, out)
    }
}

impl Backend for HipBackend {
    type BackendTensor = HipTensor;

    fn zeros(&self, shape: Shape, target_dtype: Dtype) -> TaggedTensor<Self> {
        let mut out = ptr::null_mut();
        self.check(unsafe {
            sys::cg_zeros(self.raw(), shape.0.as_ptr(), shape.0.len() as i32, dtype_code(target_dtype.clone()), &mut out)
        });
        Self::tag(matches!(target_dtype, Dtype::F32), out)
    }

    fn ndarray_from_vec_f32(&self, data: Vec<f32>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        let mut out = ptr::null_mut();
        let st = unsafe {
            sys::cg_from_f32(self.raw(), data.as_ptr(), data.len(), shape.0.as_ptr(), shape.0.len() as i32, &mut out)
        };
        if st == sys::CG_ERR_SHAPE {
            return Err(BackendError::ShapeError);
        }
        self.check(st);
        Ok(Self::tag(true, out))
    }

    fn ndarray_from_vec_u32(&self, data: Vec<u32>, shape: Shape) -> Result<TaggedTensor<Self>, BackendError> {
        let mut out = ptr::null_mut();
        let st = unsafe {
            sys::cg_from_u32(self.raw(), data.as_ptr(), data.len(), shape.0.as_ptr(), shape.0.len() as i32, &mut out)
        };
        if st == sys::CG_ERR_SHAPE {
            return Err(BackendError::ShapeError);
        }
        self.check(st);
        Ok(Self::tag(false, out))
    }

    fn cast(&self, x: TaggedTensor<Self>, target_dtype: Dtype) -> TaggedTensor<Self> {
        let (_, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_cast(self.raw(), t.0, dtype_code(target_dtype.clone()), &mut out) });
        Self::tag(matches!(target_dtype, Dtype::F32), out)
    }

    fn matmul(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_matmul, lhs)
    }
    fn add(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_add, lhs)
    }
    fn sub(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_sub, lhs)
    }
    fn mul(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_mul, lhs)
    }
    fn div(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_div, lhs)
    }
    fn pow(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_pow, lhs)
    }
    fn lt(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_lt, lhs)
    }
    fn eq(&self, lhs: TaggedTensorTuple<Self, 2>) -> TaggedTensor<Self> {
        self.binary(sys::cg_eq, lhs)
    }

    fn sin(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.unary(sys::cg_sin, x)
    }
    fn cos(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.unary(sys::cg_cos, x)
    }
    fn neg(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.unary(sys::cg_neg, x)
    }

    fn broadcast(&self, x: TaggedTensor<Self>, shape: Shape) -> TaggedTensor<Self> {
        let (is_f32, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_broadcast(self.raw(), t.0, shape.0.as_ptr(), shape.0.len() as i32, &mut out) });
        Self::tag(is_f32, out)
    }

    fn reshape(&self, x: TaggedTensor<Self>, new_shape: Shape) -> TaggedTensor<Self> {
        let (is_f32, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_reshape(self.raw(), t.0, new_shape.0.as_ptr(), new_shape.0.len() as i32, &mut out) });
        Self::tag(is_f32, out)
    }

    fn transpose(&self, x: TaggedTensor<Self>, dim0: usize, dim1: usize) -> TaggedTensor<Self> {
        let (is_f32, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_transpose(self.raw(), t.0, dim0, dim1, &mut out) });
        Self::tag(is_f32, out)
    }

    fn max(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.unary(sys::cg_max, x)
    }
    fn sum(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        self.unary(sys::cg_sum, x)
    }

    /// always U32, rank kept (ndarray.rs:240-246)
    fn argmax(&self, x: TaggedTensor<Self>) -> TaggedTensor<Self> {
        let (_, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_argmax(self.raw(), t.0, &mut out) });
        Self::tag(false, out)
    }

    /// (values F32, indices U32); F32 input only (ndarray.rs:248-257)
    fn topk(&self, x: TaggedTensor<Self>, k: usize) -> (TaggedTensor<Self>, TaggedTensor<Self>) {
        let (_, t) = Self::untag(x);
        let (mut values, mut indices) = (ptr::null_mut(), ptr::null_mut());
        self.check(unsafe { sys::cg_topk(self.raw(), t.0, k, &mut values, &mut indices) });
        (Self::tag(true, values), Self::tag(false, indices))
    }

    /// waits for the device
    fn compare(&self, x: TaggedTensorTuple<Self, 2>) -> bool {
        let [a, b] = match x {
            TaggedTensorTuple::F32(t) => t,
            TaggedTensorTuple::U32(t) => t,
        };
        let mut equal = 0;
        self.check(unsafe { sys::cg_compare(self.raw(), a.0, b.0, &mut equal) });
        equal != 0
    }

    fn concat(&self, x: TaggedTensor<Self>, y: TaggedTensor<Self>, dim: usize) -> TaggedTensor<Self> {
        let (is_f32, a) = Self::untag(x);
        let (_, b) = Self::untag(y);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_concat(self.raw(), a.0, b.0, dim, &mut out) });
        Self::tag(is_f32, out)
    }

    /// indices of any rank are used in their flattened order (ndarray.rs:373-381)
    fn index(&self, x: TaggedTensor<Self>, dim: usize, indices: TaggedTensor<Self>) -> TaggedTensor<Self> {
        let (is_f32, t) = Self::untag(x);
        let (_, idx) = Self::untag(indices);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_index(self.raw(), t.0, dim, idx.0, &mut out) });
        Self::tag(is_f32, out)
    }

    fn slice(&self, x: TaggedTensor<Self>, dim: usize, start: usize, len: usize) -> TaggedTensor<Self> {
        let (is_f32, t) = Self::untag(x);
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_slice(self.raw(), t.0, dim, start, len, &mut out) });
        Self::tag(is_f32, out)
    }

    fn arange(&self, end: usize) -> TaggedTensor<Self> {
        let mut out = ptr::null_mut();
        self.check(unsafe { sys::cg_arange(self.raw(), end, &mut out) });
        Self::tag(false, out)
    }

    /// the device -> host copy: waits for the work the value depends on
    fn to_vec(&self, vec: TaggedTensor<Self>) -> TaggedVec {
        let (is_f32, t) = Self::untag(vec);
        let n = unsafe { sys::cg_tensor_size(t.0) };
        if is_f32 {
            let mut data = vec![0f32; n];
            self.check(unsafe { sys::cg_to_f32(self.raw(), t.0, data.as_mut_ptr(), n) });
            TaggedVec::F32(data)
        } else {
            let mut data = vec![0u32; n];
            self.check(unsafe { sys::cg_to_u32(self.raw(), t.0, data.as_mut_ptr(), n) });
            TaggedVec::U32(data)
        }
    }
}

#[cfg(test)]
mod tests {
    use super::*;

    /// catgrad/src/interpreter/backend/ndarray.rs:631-674, on the device
    #[test]
    fn test_batched_matmul() {
        let backend = HipBackend::new(0, false);
        let lhs: Vec<f32> = (1..=24).map(|v| v as f32).collect();
        let rhs: Vec<f32> = (1..=12).map(|v| v as f32).collect();
        let a = backend.ndarray_from_vec_f32(lhs, Shape(vec![2, 3, 2, 2])).unwrap();
        let b = backend.ndarray_from_vec_f32(rhs, Shape(vec![2, 3, 2, 1])).unwrap();
        let (TaggedTensorTuple::F32([a]), TaggedTensorTuple::F32([b])) = (a, b) else { panic!() };
        let c = backend.matmul(TaggedTensorTuple::F32([a, b]));
        assert_eq!(c.shape(), Shape(vec![2, 3, 2, 1]));
        let TaggedVec::F32(v) = backend.to_vec(c) else { panic!() };
        assert_eq!(v, vec![5., 11., 39., 53., 105., 127., 203., 233., 333., 371., 495., 541.]);
    }

    #[test]
    fn test_shape_error() {
        let backend = HipBackend::new(0, false);
        assert!(backend.ndarray_from_vec_u32(vec![1, 2, 3], Shape(vec![2, 2])).is_err());
    }
}

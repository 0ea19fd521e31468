"""ctypes binding of include/catgrad_hip.h.

`Backend` mirrors `trait Backend` (catgrad/src/interpreter/backend/mod.rs:22-82) method for
method, with the reference's names and argument order.  Where the reference panics the binding
raises `BackendPanic`; where it returns `Err(BackendError::ShapeError)` it raises `ShapeError`.
The same binding drives the HIP library (the product) and the CPU oracle (tests only): both
export the same symbols.
"""
import ctypes as C
import os

import numpy as np

F32, U32 = 0, 1
FLAG_BF16, FLAG_EAGER, FLAG_NO_PATTERNS, FLAG_ATTN_ONE_PASS = 1, 2, 4, 8
MAX_RANK = 8

OK, ERR_SHAPE, ERR_DTYPE, ERR_ARG, ERR_DEVICE, ERR_OOM, ERR_ARITH, ERR_INTERNAL = range(8)
ERR_MULTIPLE_READ, ERR_MULTIPLE_WRITE, ERR_CYCLE, ERR_TYPE, ERR_ARITY, ERR_LOAD, ERR_APPLY = range(20, 27)

HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIB = os.path.join(HERE, "csrc", "libcatgrad_hip.so")


class BackendPanic(RuntimeError):
    """A condition on which the reference backend panics."""

    def __init__(self, status, message):
        super().__init__(f"[status {status}] {message}")
        self.status = status
        self.message = message


class ShapeError(BackendPanic):
    """BackendError::ShapeError (backend/mod.rs:88-92) and shape-mismatch panics."""


class InterpreterError(RuntimeError):
    """abstract_interpreter::InterpreterError (types.rs:95-112)."""

    def __init__(self, status, message, ident):
        super().__init__(f"[status {status}] {message}")
        self.status = status
        self.message = message
        self.ident = ident


class cg_value(C.Structure):
    _fields_ = [("kind", C.c_int), ("nat", C.c_size_t), ("dtype", C.c_int), ("rank", C.c_int),
                ("dims", C.c_size_t * MAX_RANK), ("tensor", C.c_void_p)]


_P, _PP = C.c_void_p, C.POINTER(C.c_void_p)
_SZ, _SZP = C.c_size_t, C.POINTER(C.c_size_t)
_U32P = C.POINTER(C.c_uint32)

_BIN = ["add", "sub", "mul", "div", "pow", "lt", "eq", "matmul"]
_UN = ["sin", "cos", "neg", "max", "sum", "argmax"]

_SIGNATURES = {
    "cg_backend_create": (C.c_int, [C.c_int, C.c_uint32, _PP]),
    "cg_backend_destroy": (None, [_P]),
    "cg_last_error": (C.c_char_p, [_P]),
    "cg_sync": (C.c_int, [_P]),
    "cg_tensor_realize": (C.c_int, [_P, _P]),
    "cg_tensor_prefetch": (C.c_int, [_P, _P]),
    "cg_peak_copy_gbs": (C.c_int, [_P, _SZ, C.c_int, C.POINTER(C.c_double)]),
    "cg_peak_mfma_tflops": (C.c_int, [_P, C.c_int, C.c_int, C.POINTER(C.c_double)]),
    "cg_peak_gemm_clock": (C.c_int, [_P, _SZ, _SZ, _SZ, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "cg_backend_name": (C.c_char_p, [_P]),
    "cg_tensor_retain": (_P, [_P]),
    "cg_tensor_release": (None, [_P]),
    "cg_tensor_rank": (C.c_int, [_P]),
    "cg_tensor_shape": (C.c_int, [_P, _SZP]),
    "cg_tensor_dtype": (C.c_int, [_P]),
    "cg_tensor_size": (_SZ, [_P]),
    "cg_zeros": (C.c_int, [_P, _SZP, C.c_int, C.c_int, _PP]),
    "cg_from_f32": (C.c_int, [_P, _P, _SZ, _SZP, C.c_int, _PP]),
    "cg_from_u32": (C.c_int, [_P, _P, _SZ, _SZP, C.c_int, _PP]),
    "cg_cast": (C.c_int, [_P, _P, C.c_int, _PP]),
    "cg_broadcast": (C.c_int, [_P, _P, _SZP, C.c_int, _PP]),
    "cg_reshape": (C.c_int, [_P, _P, _SZP, C.c_int, _PP]),
    "cg_transpose": (C.c_int, [_P, _P, _SZ, _SZ, _PP]),
    "cg_argmax_into": (C.c_int, [_P, _P, _P]),
    "cg_topk": (C.c_int, [_P, _P, _SZ, _PP, _PP]),
    "cg_compare": (C.c_int, [_P, _P, _P, C.POINTER(C.c_int)]),
    "cg_concat": (C.c_int, [_P, _P, _P, _SZ, _PP]),
    "cg_index": (C.c_int, [_P, _P, _SZ, _P, _PP]),
    "cg_slice": (C.c_int, [_P, _P, _SZ, _SZ, _SZ, _PP]),
    "cg_arange": (C.c_int, [_P, _SZ, _PP]),
    "cg_to_f32": (C.c_int, [_P, _P, _P, _SZ]),
    "cg_to_u32": (C.c_int, [_P, _P, _P, _SZ]),
    "cg_trace_enable": (C.c_int, [_P, C.c_int]),
    "cg_trace_reset": (C.c_int, [_P]),
    "cg_trace_report": (_SZ, [_P, C.c_char_p, _SZ]),
    "cg_launch_counts": (_SZ, [_P, C.c_int, C.c_char_p, _SZ]),
    "cg_stats": (C.c_int, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "cg_term_create": (C.c_int, [_PP]),
    "cg_term_destroy": (None, [_P]),
    "cg_term_add_node": (C.c_int, [_P, C.c_int, _U32P]),
    "cg_term_add_op": (C.c_int, [_P, C.c_int, C.c_char_p, C.c_uint64, _U32P, _SZ, _U32P, _SZ, _U32P]),
    "cg_term_set_boundary": (C.c_int, [_P, _U32P, _SZ, _U32P, _SZ]),
    "cg_term_stats": (C.c_int, [_P, _SZP, _SZP]),
    "cg_env_create": (C.c_int, [_PP]),
    "cg_env_destroy": (None, [_P]),
    "cg_env_define": (C.c_int, [_P, C.c_char_p, _P]),
    "cg_params_create": (C.c_int, [_PP]),
    "cg_params_destroy": (None, [_P]),
    "cg_params_set": (C.c_int, [_P, C.c_char_p, _P]),
    "cg_params_len": (_SZ, [_P]),
    "cg_params_key": (C.c_char_p, [_P, _SZ]),
    "cg_params_get": (C.c_int, [_P, C.c_char_p, _PP]),
    "cg_params_remove": (C.c_int, [_P, C.c_char_p]),
    "cg_from_bf16": (C.c_int, [_P, _P, _SZ, _SZP, C.c_int, _PP]),
    "cg_stack": (C.c_int, [_P, _PP, _SZ, _PP]),
    "cg_weights_open": (C.c_int, [C.c_char_p, _PP]),
    "cg_weights_close": (None, [_P]),
    "cg_weights_count": (_SZ, [_P]),
    "cg_weights_name": (C.c_char_p, [_P, _SZ]),
    "cg_weights_info": (C.c_int, [_P, _SZ, C.POINTER(C.c_int), C.POINTER(C.c_char_p), C.POINTER(C.c_int), _SZP,
                                  C.POINTER(C.c_uint64)]),
    "cg_weights_tensor": (C.c_int, [_P, _P, _SZ, _PP]),
    "cg_params_load": (C.c_int, [_P, _P, C.c_char_p, C.c_char_p, _SZP]),
    "cg_params_stack_experts": (C.c_int, [_P, _P, C.c_char_p, _SZ, _SZ]),
    "cg_weights_last_error": (C.c_char_p, []),
    "cg_interp_eval": (C.c_int, [_P, _P, _P, _P, C.POINTER(cg_value), _SZ, C.POINTER(cg_value), _SZ, _U32P]),
    "cg_interp_eval_owned": (C.c_int, [_P, _P, _P, _P, C.POINTER(cg_value), _SZ, C.POINTER(cg_value), _SZ, _U32P]),
    "cg_interp_last_error": (C.c_char_p, []),
    "cg_interp_backend_calls": (C.c_uint64, [C.c_int]),
}
for _n in _BIN:
    _SIGNATURES["cg_" + _n] = (C.c_int, [_P, _P, _P, _PP])
for _n in _UN:
    _SIGNATURES["cg_" + _n] = (C.c_int, [_P, _P, _PP])

EXPORTED_SYMBOLS = sorted(_SIGNATURES)


def load_library(path=None):
    """dlopen a library exporting the catgrad_hip.h ABI and declare its signatures."""
    path = path or HIP_LIB
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
    lib = C.CDLL(path, mode=C.RTLD_LOCAL)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    lib._path = path
    return lib


def _dims(shape):
    shape = tuple(int(d) for d in shape)
    if len(shape) > MAX_RANK:
        raise ShapeError(ERR_ARG, f"rank {len(shape)} above {MAX_RANK}")
    return (C.c_size_t * max(len(shape), 1))(*shape), len(shape)


class Tensor:
    """A BackendTensor handle (ref-counted, O(1) clone) with its dtype tag."""

    __slots__ = ("_lib", "_be", "ptr")

    def __init__(self, be, ptr):
        self._be = be
        self._lib = be.lib
        self.ptr = ptr

    def __del__(self):
        if getattr(self, "ptr", None):
            self._lib.cg_tensor_release(self.ptr)
            self.ptr = None

    def clone(self):
        return Tensor(self._be, self._lib.cg_tensor_retain(self.ptr))

    @property
    def shape(self):
        """BackendTensorOps::shape (backend/mod.rs:84-86)."""
        r = self._lib.cg_tensor_rank(self.ptr)
        d = (C.c_size_t * max(r, 1))()
        self._lib.cg_tensor_shape(self.ptr, d)
        return tuple(d[i] for i in range(r))

    @property
    def dtype(self):
        return self._lib.cg_tensor_dtype(self.ptr)

    def __repr__(self):
        return f"Tensor({'F32' if self.dtype == F32 else 'U32'}, {list(self.shape)})"


class Backend:
    """`impl Backend` over the C ABI: one instance = one device + one stream."""

    def __init__(self, lib=None, device=0, flags=0):
        self.lib = lib if lib is not None else load_library()
        p = C.c_void_p()
        st = self.lib.cg_backend_create(device, flags, C.byref(p))
        if st:
            raise BackendPanic(st, "cg_backend_create failed (no usable GPU?)")
        self.ptr = p
        self.flags = flags

    def close(self):
        """Give the backend up now (its launch thread is joined, its stream and pool released once the
        last tensor of it is gone) instead of whenever the garbage collector finds the object."""
        if getattr(self, "ptr", None):
            self.lib.cg_backend_destroy(self.ptr)
            self.ptr = None

    def __del__(self):
        # tensors may outlive the Python object; the library keeps the backend alive for them
        self.close()

    @property
    def name(self):
        return self.lib.cg_backend_name(self.ptr).decode()

    # -- plumbing ------------------------------------------------------------------
    def _check(self, st):
        if st:
            msg = self.lib.cg_last_error(self.ptr).decode(errors="replace")
            raise (ShapeError if st == ERR_SHAPE else BackendPanic)(st, msg)

    def _out(self, fn, *args):
        out = C.c_void_p()
        self._check(fn(self.ptr, *args, C.byref(out)))
        return Tensor(self, out.value)

    def sync(self):
        self._check(self.lib.cg_sync(self.ptr))

    def peak_copy_gbs(self, nbytes=1 << 30, iters=10):
        out = C.c_double()
        self._check(self.lib.cg_peak_copy_gbs(self.ptr, nbytes, iters, C.byref(out)))
        return out.value

    def peak_mfma_tflops(self, operand=None, iters=20000):
        out = C.c_double()
        self._check(self.lib.cg_peak_mfma_tflops(self.ptr, U32 if operand is None else operand, iters, C.byref(out)))
        return out.value

    def peak_gemm_clock(self, m, n, k, iters=5):
        """(TFLOP/s, shader clock in MHz) of the bf16 GEMM m x n x k; m == 0: of the register-resident MFMA loop."""
        tf, mhz = C.c_double(), C.c_double()
        self._check(self.lib.cg_peak_gemm_clock(self.ptr, m, n, k, iters, C.byref(tf), C.byref(mhz)))
        return tf.value, mhz.value

    def prefetch(self, x):
        """Realize and start an asynchronous copy of a small tensor to the host; `to_vec(x)` then
        waits for that copy alone."""
        self._check(self.lib.cg_tensor_prefetch(self.ptr, x.ptr))
        return x

    def realize(self, x):
        """Issue the kernels a deferred tensor still needs (no wait)."""
        self._check(self.lib.cg_tensor_realize(self.ptr, x.ptr))
        return x

    # -- trait methods -----------------------------------------------------------------
    def zeros(self, shape, target_dtype):
        d, r = _dims(shape)
        return self._out(self.lib.cg_zeros, d, r, target_dtype)

    def ndarray_from_vec_f32(self, data, shape):
        a = np.ascontiguousarray(data, dtype=np.float32).reshape(-1)
        d, r = _dims(shape)
        return self._out(self.lib.cg_from_f32, a.ctypes.data, a.size, d, r)

    def ndarray_from_vec_u32(self, data, shape):
        a = np.ascontiguousarray(data, dtype=np.uint32).reshape(-1)
        d, r = _dims(shape)
        return self._out(self.lib.cg_from_u32, a.ctypes.data, a.size, d, r)

    def from_bf16_bits(self, bits, shape):
        """An F32 tensor from bf16 bit patterns (uint16), widened by the backend."""
        a = np.ascontiguousarray(bits, dtype=np.uint16).reshape(-1)
        d, r = _dims(shape)
        return self._out(self.lib.cg_from_bf16, a.ctypes.data, a.size, d, r)

    def stack(self, parts):
        """[n, ...] from n tensors of one shape."""
        arr = (C.c_void_p * len(parts))(*[t.ptr for t in parts])
        return self._out(self.lib.cg_stack, arr, len(parts))

    def cast(self, x, target_dtype):
        return self._out(self.lib.cg_cast, x.ptr, target_dtype)

    def broadcast(self, x, shape):
        d, r = _dims(shape)
        return self._out(self.lib.cg_broadcast, x.ptr, d, r)

    def reshape(self, x, new_shape):
        d, r = _dims(new_shape)
        return self._out(self.lib.cg_reshape, x.ptr, d, r)

    def transpose(self, x, dim0, dim1):
        return self._out(self.lib.cg_transpose, x.ptr, dim0, dim1)

    def argmax_into(self, x, out):
        """argmax of `x` into the tensor `out` (both already in memory); allocates nothing."""
        self._check(self.lib.cg_argmax_into(self.ptr, x.ptr, out.ptr))
        return out

    def topk(self, x, k):
        v, i = C.c_void_p(), C.c_void_p()
        self._check(self.lib.cg_topk(self.ptr, x.ptr, k, C.byref(v), C.byref(i)))
        return Tensor(self, v.value), Tensor(self, i.value)

    def compare(self, a, b):
        eq = C.c_int(0)
        self._check(self.lib.cg_compare(self.ptr, a.ptr, b.ptr, C.byref(eq)))
        return bool(eq.value)

    def concat(self, x, y, dim):
        return self._out(self.lib.cg_concat, x.ptr, y.ptr, dim)

    def index(self, x, dim, indices):
        return self._out(self.lib.cg_index, x.ptr, dim, indices.ptr)

    def slice(self, x, dim, start, len):  # noqa: A002 - the reference's parameter name
        return self._out(self.lib.cg_slice, x.ptr, dim, start, len)

    def arange(self, end):
        return self._out(self.lib.cg_arange, end)

    def to_vec(self, x):
        """to_vec (mod.rs:81): a flat numpy array, float32 or uint32 by the tensor's tag."""
        n = self.lib.cg_tensor_size(x.ptr)
        if x.dtype == F32:
            a = np.empty(n, dtype=np.float32)
            self._check(self.lib.cg_to_f32(self.ptr, x.ptr, a.ctypes.data, n))
        else:
            a = np.empty(n, dtype=np.uint32)
            self._check(self.lib.cg_to_u32(self.ptr, x.ptr, a.ctypes.data, n))
        return a

    # -- conveniences (not in the trait) ----------------------------------------------
    def tensor(self, data, shape=None):
        """interpreter::tensor (interpreter/mod.rs:21-31) from a numpy array."""
        a = np.asarray(data)
        shape = a.shape if shape is None else shape
        if a.dtype == np.uint32:
            return self.ndarray_from_vec_u32(a, shape)
        return self.ndarray_from_vec_f32(a, shape)

    def numpy(self, x):
        return self.to_vec(x).reshape(x.shape)

    def trace(self, on):
        self._check(self.lib.cg_trace_enable(self.ptr, int(on)))

    def trace_reset(self):
        self._check(self.lib.cg_trace_reset(self.ptr))

    def trace_report(self):
        """{kernel name: {"launches", "ms", "bytes", "flops"}} since the last reset."""
        n = self.lib.cg_trace_report(self.ptr, None, 0)
        buf = C.create_string_buffer(n + 1)
        self.lib.cg_trace_report(self.ptr, buf, n + 1)
        rep = {}
        for line in buf.value.decode().splitlines():
            f = line.split()
            if len(f) == 5:
                rep[f[0]] = {"launches": int(f[1]), "ms": float(f[2]), "bytes": float(f[3]),
                             "flops": float(f[4])}
        return rep

    def launch_counts(self, reset=False):
        """{kernel family: launches} since creation or the last reset (no tracing needed)."""
        n = self.lib.cg_launch_counts(self.ptr, 0, None, 0)
        buf = C.create_string_buffer(n + 1)
        self.lib.cg_launch_counts(self.ptr, int(reset), buf, n + 1)
        out = {}
        for line in buf.value.decode().splitlines():
            name, cnt = line.rsplit(" ", 1)
            if int(cnt):
                out[name] = int(cnt)
        return out

    GENERIC_PROGRAMS = ("ew_fused", "row_fused")

    def stats(self):
        a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
        self.lib.cg_stats(self.ptr, C.byref(a), C.byref(b), C.byref(c))
        return {"launches": a.value, "device_bytes": b.value, "pool_bytes": c.value}


def _make_bin(name):
    def f(self, a, b):
        return self._out(getattr(self.lib, "cg_" + name), a.ptr, b.ptr)
    f.__name__ = name
    return f


def _make_un(name):
    def f(self, x):
        return self._out(getattr(self.lib, "cg_" + name), x.ptr)
    f.__name__ = name
    return f


for _n in _BIN:
    setattr(Backend, _n, _make_bin(_n))
for _n in _UN:
    setattr(Backend, _n, _make_un(_n))

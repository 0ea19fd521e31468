"""`Interpreter`, `Environment`, `Parameters`, `Value`: the caller's side of the evaluator.

Mirror of catgrad/src/interpreter/{interpreter,types,mod}.rs.  Evaluation itself is native
(csrc/interp.cpp behind cg_interp_eval); this module only marshals values.
"""
import ctypes as C
import os

import numpy as np

from . import abi
from .lang import Term
from .nn import stdlib_definitions

VAL_NAT, VAL_DTYPE, VAL_SHAPE, VAL_TENSOR = 0, 1, 2, 4


class Nat(int):
    """Value::Nat"""


class Dtype(int):
    """Value::Dtype"""


class Shape(tuple):
    """Value::Shape / core::Shape"""

    def size(self):
        n = 1
        for d in self:
            n *= d
        return n


class Environment:
    """pass::to_core::Environment: definitions by path (declarations are fixed, lang.py)."""

    def __init__(self, modules=()):
        self.definitions = {}
        self._handles = {}
        for m in modules:
            self.define(m)

    def define(self, module):
        self.definitions[str(module.path())] = module.term()
        self._handles.clear()

    def handle(self, lib):
        key = lib._path
        if key not in self._handles:
            e = C.c_void_p()
            lib.cg_env_create(C.byref(e))
            terms = []
            for p, t in self.definitions.items():
                h = t.compile(lib)
                terms.append(h)
                lib.cg_env_define(e, p.encode(), h.ptr)
            self._handles[key] = _Owned(lib.cg_env_destroy, e, terms)
        return self._handles[key]


def stdlib():
    """stdlib_definitions.rs:35-40"""
    return Environment(stdlib_definitions())


class WeightsError(RuntimeError):
    """A weight file could not be read (the reference's loader returns Err or panics)."""

    def __init__(self, status, message):
        super().__init__(f"[{status}] {message}")
        self.status, self.message = status, message


class Parameters(dict):
    """abstract_interpreter::parameters::Parameters: path -> tensor Value."""

    def handle(self, lib):
        p = C.c_void_p()
        lib.cg_params_create(C.byref(p))
        for k, v in self.items():
            lib.cg_params_set(p, str(k).encode(), v.ptr)
        return _Owned(lib.cg_params_destroy, p, None)

    def _take(self, backend, native):
        """Replace the contents by those of a native table."""
        lib = backend.lib
        self.clear()
        for i in range(lib.cg_params_len(native.ptr)):
            key = lib.cg_params_key(native.ptr, i)
            t = C.c_void_p()
            lib.cg_params_get(native.ptr, key, C.byref(t))
            self[key.decode()] = abi.Tensor(backend, t.value)

    def load_safetensors(self, backend, files, prefix=""):
        """The loading loop of catgrad-llm/examples/llama/main.rs:288-333, natively: every tensor of
        every file becomes the parameter prefix + name (F32 and BF16 files only)."""
        lib = backend.lib
        native = self.handle(lib)
        for f in ([files] if isinstance(files, (str, bytes, os.PathLike)) else files):
            n = C.c_size_t()
            st = lib.cg_params_load(backend.ptr, native.ptr, str(f).encode(), prefix.encode(), C.byref(n))
            if st:
                raise WeightsError(st, lib.cg_weights_last_error().decode(errors="replace"))
        self._take(backend, native)
        return self

    def stack_experts(self, backend, num_layers, num_experts, prefix=""):
        """concat_moe_experts (main.rs:171-262): per layer and projection, the experts' matrices
        become one [E, ...] parameter."""
        lib = backend.lib
        native = self.handle(lib)
        st = lib.cg_params_stack_experts(backend.ptr, native.ptr, prefix.encode(), num_layers, num_experts)
        if st:
            raise WeightsError(st, lib.cg_weights_last_error().decode(errors="replace"))
        self._take(backend, native)
        return self


class WeightFile:
    """An open safetensors file: names, dtypes and shapes from the header (host only)."""

    def __init__(self, lib, path):
        self.lib, self.ptr = lib, None
        w = C.c_void_p()
        st = lib.cg_weights_open(str(path).encode(), C.byref(w))
        if st:
            raise WeightsError(st, lib.cg_weights_last_error().decode(errors="replace"))
        self.ptr = w

    def close(self):
        if self.ptr:
            self.lib.cg_weights_close(self.ptr)
            self.ptr = None

    __del__ = close

    def __len__(self):
        return self.lib.cg_weights_count(self.ptr)

    def entries(self):
        """[(name, dtype string, shape tuple, byte count)] in header order."""
        out = []
        for i in range(len(self)):
            dt, name, rank, nbytes = C.c_int(), C.c_char_p(), C.c_int(), C.c_uint64()
            dims = (C.c_size_t * 8)()
            self.lib.cg_weights_info(self.ptr, i, C.byref(dt), C.byref(name), C.byref(rank), dims, C.byref(nbytes))
            out.append((self.lib.cg_weights_name(self.ptr, i).decode(), name.value.decode(),
                        tuple(dims[d] for d in range(rank.value)), nbytes.value))
        return out

    def tensor(self, backend, i):
        t = C.c_void_p()
        st = self.lib.cg_weights_tensor(backend.ptr, self.ptr, i, C.byref(t))
        if st:
            raise WeightsError(st, self.lib.cg_weights_last_error().decode(errors="replace"))
        return abi.Tensor(backend, t.value)


class _Owned:
    def __init__(self, destroy, ptr, keep):
        self.destroy, self.ptr, self.keep = destroy, ptr, keep

    def __del__(self):
        if self.ptr:
            self.destroy(self.ptr)
            self.ptr = None


def tensor(backend, shape, data):
    """interpreter::tensor (interpreter/mod.rs:21-31): ShapeError unless sizes agree."""
    a = np.asarray(data)
    if Shape(shape).size() != a.size:
        raise abi.ShapeError(abi.ERR_SHAPE, "ShapeError")
    if a.dtype == np.uint32 or (a.dtype.kind in "iu" and a.dtype != np.float32):
        return backend.ndarray_from_vec_u32(a.astype(np.uint32), shape)
    return backend.ndarray_from_vec_f32(a, shape)


class Interpreter:
    """interpreter.rs:14-37"""

    def __init__(self, backend, environment, parameters=None):
        self.backend = backend
        self.environment = environment
        self.parameters = parameters if parameters is not None else Parameters()
        self._params_handle = None
        self._params_len = -1

    def _params(self):
        if self._params_handle is None or self._params_len != len(self.parameters):
            self._params_handle = self.parameters.handle(self.backend.lib)
            self._params_len = len(self.parameters)
        return self._params_handle

    def run(self, term, args, moved=()):
        """Interpreter::run: `args` are Tensor / Nat / Dtype / Shape values; returns the same.
        `moved`: positions of tensor arguments given away, as the Rust `run` takes its values by
        value: those Tensor objects are empty afterwards (KV-cache tensors are passed this way so
        that the step may append to them in place)."""
        assert isinstance(term, Term)
        lib = self.backend.lib
        h = term.compile(lib)
        n_out = len(term.targets)
        cargs = (abi.cg_value * max(len(args), 1))()
        for i, a in enumerate(args):
            v = cargs[i]
            if isinstance(a, abi.Tensor):
                v.kind, v.tensor = VAL_TENSOR, a.ptr
                if i in moved:
                    a.ptr = None                    # the evaluator takes over this reference
                else:
                    lib.cg_tensor_retain(v.tensor)  # the owned call consumes one reference per tensor
            elif isinstance(a, Shape) or isinstance(a, (tuple, list)):
                v.kind, v.rank = VAL_SHAPE, len(a)
                for j, d in enumerate(a):
                    v.dims[j] = d
            elif isinstance(a, Dtype):
                v.kind, v.dtype = VAL_DTYPE, int(a)
            else:
                v.kind, v.nat = VAL_NAT, int(a)
        res = (abi.cg_value * max(n_out, 1))()
        err_id = C.c_uint32(0)
        moved = frozenset(moved)
        st = lib.cg_interp_eval_owned(self.backend.ptr, self.environment.handle(lib).ptr,
                                self._params().ptr, h.ptr, cargs, len(args), res, n_out,
                                C.byref(err_id))
        if st:
            msg = lib.cg_interp_last_error().decode(errors="replace")
            if st < 20:
                raise (abi.ShapeError if st == abi.ERR_SHAPE else abi.BackendPanic)(st, msg)
            raise abi.InterpreterError(st, msg, err_id.value)
        out = []
        for i in range(n_out):
            v = res[i]
            if v.kind == VAL_TENSOR:
                out.append(abi.Tensor(self.backend, v.tensor))
            elif v.kind == VAL_SHAPE:
                out.append(Shape(v.dims[j] for j in range(v.rank)))
            elif v.kind == VAL_DTYPE:
                out.append(Dtype(v.dtype))
            else:
                out.append(Nat(v.nat))
        return out

    def backend_calls(self, reset=True):
        return self.backend.lib.cg_interp_backend_calls(int(reset))

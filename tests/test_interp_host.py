"""Host logic: the native evaluator's rules (eval.rs / tensor_op.rs) and error reporting,
driven on the CPU oracle; and that the product library exports the whole C ABI."""
import ctypes
import os
import re

import numpy as np
import pytest

import vectors

lang = vectors.lang
T, N, S = lang.TENSOR, lang.NAT, lang.SHAPE


def test_hip_library_exports_every_declared_symbol(cg):
    """include/catgrad_hip.h <-> libcatgrad_hip.so <-> abi.py agree (no compute calls)."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    header = open(os.path.join(root, "include", "catgrad_hip.h")).read()
    declared = set(re.findall(r"\b(cg_[a-z0-9_]+)\s*\(", header))
    declared -= {"cg_value", "cg_object", "cg_dtype", "cg_opcode", "cg_value_kind"}
    assert declared == set(cg.abi.EXPORTED_SYMBOLS)
    lib = ctypes.CDLL(cg.abi.HIP_LIB)
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} missing from libcatgrad_hip.so"
    olib = ctypes.CDLL(os.path.join(root, "oracle", "liboracle.so"))
    for name in sorted(declared):
        assert hasattr(olib, name), f"{name} missing from liboracle.so"


def test_product_fails_loudly_without_gpu(cg):
    import torch  # noqa: F401 - only to ask whether this host has a GPU
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(cg.BackendPanic):
        cg.Backend(cg.load_library())


def test_copy_fanout_and_discard(oracle, cg):
    def f(b, x):
        sh = lang.shape(b, x)
        _a, _b = lang.unpack(b, 2, sh)          # both discarded
        return x + x * x, x
    t = vectors.Fn("f", 1, 2, f).term()
    nodes, edges, src, tgt = t.lowered()
    copies = [e for e in edges if e[0] == lang.OP_COPY]
    assert any(len(e[4]) == 5 for e in copies)          # x read five times
    assert sum(len(e[4]) == 0 for e in copies) == 2     # two discarded Nats
    x = np.arange(6, dtype=np.float32).reshape(2, 3)
    y, x2 = vectors.run(oracle, f, 2, x)
    assert np.array_equal(y, x + x * x) and np.array_equal(x2, x)
    assert t.stats(oracle.lib)["ops"] == len(edges)


def test_nat_shape_dtype_values(oracle, cg):
    it = cg.Interpreter(oracle, cg.stdlib())

    class M(lang.Module):
        def path(self):
            return lang.path(["test", "values"])

        def sort(self):
            return [T, N], [S, N, lang.DTYPE, T]

        def def_(self, b, args):
            x, n = args
            sh = lang.shape(b, x)
            a, c = lang.unpack(b, 2, sh)
            return [lang.pack(b, [c, a, n]), a * c + n, lang.dtype(b, x), lang.nat_to_u32(b, n)]
    x = oracle.tensor(np.zeros((2, 5), np.uint32))
    sh, n, dt, t = it.run(M().term(), [x, 7])
    assert tuple(sh) == (5, 2, 7) and n == 17 and dt == cg.U32
    assert t.shape == () and t.dtype == cg.U32 and oracle.to_vec(t)[0] == 7


def test_argument_orders(oracle):
    """tensor_op.rs: Reshape = [shape, x], Broadcast = [x, shape], Slice = [x, dim, start, len],
    Concat = [a, b, dim], Index = [x, dim, idx], Transpose = [x, d0, d1], Cast = [x, dtype]."""
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)

    def f(b, x):
        r = lang.reshape(b, lang.make_shape(b, 6, 4), x)
        t = lang.transpose(b, 0, 1, r)                              # [4, 6]
        s = lang.slice(b, 1, 2, 3, t)                               # [4, 3]
        c = lang.concat(b, 1, s, s)                                 # [4, 6]
        i = lang.index(b, 0, lang.arange(b, 2), c)                  # rows 0, 1
        bc = lang.broadcast(b, i, lang.make_shape(b, 5, 2, 6))
        return lang.cast(b, lang.cast(b, bc, lang.dtype(b, lang.arange(b, 1))), 0)
    (y,) = vectors.run(oracle, f, 1, a)
    s = a.reshape(6, 4).T[:, 2:5]
    ref = np.broadcast_to(np.concatenate([s, s], 1)[:2], (5, 2, 6))
    assert np.array_equal(y, ref)


def test_interpreter_errors(oracle, cg):
    it = cg.Interpreter(oracle, cg.stdlib())
    E = cg.InterpreterError
    f32, u32 = np.zeros((2, 2), np.float32), np.zeros((2, 2), np.uint32)
    add = vectors.Fn("add", 2, 1, lambda b, x, y: x + y).term()
    # mixed dtypes -> TypeError (tensor_op.rs:216-218)
    with pytest.raises(E) as e:
        it.run(add, [oracle.tensor(f32), oracle.tensor(u32)])
    assert e.value.status == cg.abi.ERR_TYPE
    # a Nat where a tensor is wanted -> TypeError
    with pytest.raises(E) as e:
        it.run(add, [oracle.tensor(f32), 3])
    assert e.value.status == cg.abi.ERR_TYPE
    # wrong number of values
    with pytest.raises(E) as e:
        it.run(add, [oracle.tensor(f32)])
    assert e.value.status == cg.abi.ERR_ARITY
    # missing parameter -> Load
    ld = vectors.Fn("ld", 1, 1, lambda b, x: x + lang.param(b, lang.path(["nope", "weight"]))).term()
    with pytest.raises(E, match="nope.weight") as e:
        it.run(ld, [oracle.tensor(f32)])
    assert e.value.status == cg.abi.ERR_LOAD
    # shape mismatch inside a term -> the backend's panic
    with pytest.raises(cg.ShapeError, match="Shape mismatch in operation"):
        it.run(add, [oracle.tensor(f32), oracle.tensor(np.zeros((2, 3), np.float32))])
    # tensor() size check (interpreter/mod.rs:26-28)
    with pytest.raises(cg.ShapeError):
        cg.tensor(oracle, (2, 3), np.zeros(5, np.float32))
    # unknown definition
    class Ghost(lang.Module):
        def path(self):
            return lang.path(["nn", "ghost"])

        def sort(self):
            return [T], [T]
    bad = vectors.Fn("bad", 1, 1, lambda b, x: Ghost().call(b, [x])).term()
    with pytest.raises(E, match="Definition not found"):
        it.run(bad, [oracle.tensor(f32)])


def test_raw_term_errors(oracle, cg):
    """MultipleRead / MultipleWrite / ArityError / Cycle straight through the C ABI."""
    lib = oracle.lib
    C = ctypes

    def term(nodes, ops, src, tgt):
        t = C.c_void_p()
        lib.cg_term_create(C.byref(t))
        for lab in nodes:
            lib.cg_term_add_node(t, lab, None)
        for op, s, g in ops:
            lib.cg_term_add_op(t, op, None, 0, (C.c_uint32 * max(len(s), 1))(*s), len(s),
                               (C.c_uint32 * max(len(g), 1))(*g), len(g), None)
        lib.cg_term_set_boundary(t, (C.c_uint32 * max(len(src), 1))(*src), len(src),
                                 (C.c_uint32 * max(len(tgt), 1))(*tgt), len(tgt))
        return t

    def run(t, args, n_out):
        cargs = (cg.abi.cg_value * max(len(args), 1))()
        for i, a in enumerate(args):
            cargs[i].kind, cargs[i].tensor = 4, a.ptr
        res = (cg.abi.cg_value * max(n_out, 1))()
        st = lib.cg_interp_eval(oracle.ptr, None, None, t, cargs, len(args), res, n_out, None)
        for i in range(n_out if st == 0 else 0):
            cg.Tensor(oracle, res[i].tensor)
        return st
    x = oracle.tensor(np.ones((2,), np.float32))
    # node 0 read twice without a Copy
    t = term([T, T], [(lang.OP_ADD, [0, 0], [1])], [0], [1])
    assert run(t, [x], 1) == cg.abi.ERR_MULTIPLE_READ
    # node 1 written twice
    t = term([T, T, T], [(lang.OP_NEG, [0], [1]), (lang.OP_NEG, [2], [1])], [0, 2], [1])
    assert run(t, [x, x], 1) == cg.abi.ERR_MULTIPLE_WRITE
    # add with one argument
    t = term([T, T], [(lang.OP_ADD, [0], [1])], [0], [1])
    assert run(t, [x], 1) == cg.abi.ERR_ARITY
    # a cycle: 1 -> 2 -> 1
    t = term([T, T, T], [(lang.OP_NEG, [1], [2]), (lang.OP_NEG, [2], [1])], [0], [1])
    assert run(t, [x], 1) == cg.abi.ERR_CYCLE
    n_ops, n_layers = C.c_size_t(), C.c_size_t()
    assert lib.cg_term_stats(t, C.byref(n_ops), C.byref(n_layers)) == cg.abi.ERR_CYCLE


def test_layered_order_counts(oracle):
    """ssa/mod.rs: independent ops share a layer; a chain gets one layer per op."""
    chain = vectors.Fn("c", 1, 1, lambda b, x: -(-(-x))).term()
    assert chain.stats(oracle.lib) == {"ops": 3, "layers": 3}
    wide = vectors.Fn("w", 2, 2, lambda b, x, y: (-x, -y)).term()
    assert wide.stats(oracle.lib) == {"ops": 2, "layers": 1}

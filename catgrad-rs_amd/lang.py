"""Graph-building DSL: the host-side mirror of catgrad's `lang` layer.

Same names and argument order as catgrad/src/category/lang/ops.rs and
catgrad/src/stdlib/ops.rs, so that model code reads like the reference's and emits the same
sequence of core operations.  A `Builder` records hyperedges; `Term.compile` lowers them to a
`cg_term` of the C ABI (the `to_core` step, catgrad/src/pass/to_core.rs:37-123), inserting the
explicit Copy edges the reference's Var-based builder produces for every fan-out and discard.
"""
import builtins
import ctypes as C
import struct

from . import abi

# core::Object (core.rs:69-76) / cg_object
NAT, DTYPE, TYPE, SHAPE, TENSOR = range(5)

# cg_opcode, same order as include/catgrad_hip.h
(OP_COPY, OP_LOAD, OP_DEF, OP_PACK, OP_UNPACK, OP_SHAPE, OP_DTYPE, OP_NAT_CONST, OP_NAT_MUL,
 OP_NAT_ADD, OP_DTYPE_CONST, OP_ADD, OP_SUB, OP_MUL, OP_DIV, OP_NEG, OP_POW, OP_LT, OP_EQ,
 OP_COS, OP_SIN, OP_NAT_TO_U32, OP_CAST, OP_MATMUL, OP_SCALAR_F32, OP_SCALAR_U32, OP_SUM,
 OP_MAX, OP_ARGMAX, OP_TOPK, OP_BROADCAST, OP_RESHAPE, OP_TRANSPOSE, OP_SLICE, OP_CONCAT,
 OP_ARANGE, OP_INDEX) = range(37)

# to_core.rs:85-123: declared operation name -> core operation
CORE_DECLARATIONS = {
    "cartesian.copy": OP_COPY, "tensor.add": OP_ADD, "tensor.sub": OP_SUB, "tensor.neg": OP_NEG,
    "tensor.mul": OP_MUL, "tensor.div": OP_DIV, "tensor.pow": OP_POW, "tensor.sin": OP_SIN,
    "tensor.cos": OP_COS, "tensor.lt": OP_LT, "tensor.eq": OP_EQ, "tensor.matmul": OP_MATMUL,
    "tensor.reshape": OP_RESHAPE, "tensor.transpose": OP_TRANSPOSE,
    "tensor.broadcast": OP_BROADCAST, "tensor.cast": OP_CAST, "tensor.index": OP_INDEX,
    "tensor.slice": OP_SLICE, "tensor.sum": OP_SUM, "tensor.max": OP_MAX,
    "tensor.argmax": OP_ARGMAX, "tensor.topk": OP_TOPK, "tensor.arange": OP_ARANGE,
    "tensor.concat": OP_CONCAT, "tensor.nat_to_u32": OP_NAT_TO_U32, "tensor.shape": OP_SHAPE,
    "tensor.dtype": OP_DTYPE, "shape.pack": OP_PACK, "shape.unpack": OP_UNPACK,
    "nat.add": OP_NAT_ADD, "nat.mul": OP_NAT_MUL,
}


class Path(tuple):
    """crate::path::Path: a dotted name."""

    def extend(self, parts):
        return Path(self + tuple(str(p) for p in parts))

    def __str__(self):
        return ".".join(self)


def path(parts):
    return Path(tuple(str(p) for p in parts))


class F32Lit(float):
    """Literal::F32"""


class U32Lit(int):
    """Literal::U32"""


class NatLit(int):
    """Literal::Nat"""


def nat(x):
    return NatLit(x)


class Builder:
    """Records nodes and hyperedges in creation order."""

    def __init__(self):
        self.nodes = []   # object label per node
        self.edges = []   # (opcode, path or None, scalar, [source nodes], [target nodes])

    def new_node(self, label):
        self.nodes.append(label)
        return len(self.nodes) - 1

    def operation(self, sources, result_labels, opcode, path=None, scalar=0):
        """var::operation: one hyperedge, fresh target nodes."""
        for v in sources:
            assert v.builder is self, "Var from another builder"
        targets = [self.new_node(l) for l in result_labels]
        self.edges.append((opcode, str(path) if path is not None else None, scalar,
                           [v.node for v in sources], targets))
        return [Var(self, n, l) for n, l in zip(targets, result_labels)]

    def fn_operation(self, sources, label, opcode, path=None, scalar=0):
        return self.operation(sources, [label], opcode, path, scalar)[0]


class Var:
    """open_hypergraphs::lax::var::Var with the HasAdd/HasSub/... operator impls of
    lang/ops.rs:20-72."""

    __slots__ = ("builder", "node", "label")

    def __init__(self, builder, node, label):
        self.builder, self.node, self.label = builder, node, label

    def clone(self):
        return self

    def _bin(self, other, tensor_op, nat_op=None):
        assert isinstance(other, Var) and self.label == other.label, "operand sorts differ"
        if self.label == NAT:
            assert nat_op is not None, "undefined for Nat"
            return self.builder.fn_operation([self, other], NAT, nat_op)
        assert self.label == TENSOR, f"undefined for object {self.label}"
        return self.builder.fn_operation([self, other], TENSOR, tensor_op)

    def __add__(self, o):
        return self._bin(o, OP_ADD, OP_NAT_ADD)

    def __sub__(self, o):
        return self._bin(o, OP_SUB)

    def __mul__(self, o):
        return self._bin(o, OP_MUL, OP_NAT_MUL)

    def __truediv__(self, o):
        return self._bin(o, OP_DIV)

    def __neg__(self):
        return self.builder.fn_operation([self], self.label, OP_NEG)


class Term:
    """A finished open hypergraph: a Builder's edges plus source and target nodes."""

    def __init__(self, builder, sources, targets):
        self.builder = builder
        self.sources = [v.node for v in sources]
        self.targets = [v.node for v in targets]
        self._compiled = {}

    def lowered(self):
        """Edges with explicit Copy edges for every node read more (or less) than once.

        Returns (node labels, edges, sources, targets).  The reference's lax->strict
        conversion does the same with `cartesian.copy` (lang/ops.rs:22-26), and its evaluator
        relies on it: a value is moved out of the state on its single read (eval.rs:43-49).
        """
        nodes = list(self.builder.nodes)
        edges = [(op, p, s, list(src), list(tgt)) for op, p, s, src, tgt in self.builder.edges]
        targets = list(self.targets)
        uses = {}
        for ei, e in enumerate(edges):
            for si, n in enumerate(e[3]):
                uses.setdefault(n, []).append((ei, si))
        for ti, n in enumerate(targets):
            uses.setdefault(n, []).append((-1, ti))
        copies = []
        for n in range(len(self.builder.nodes)):
            u = uses.get(n, [])
            if len(u) == 1:
                continue
            fresh = []
            for ei, si in u:
                nodes.append(nodes[n])
                m = len(nodes) - 1
                fresh.append(m)
                if ei < 0:
                    targets[si] = m
                else:
                    edges[ei][3][si] = m
            copies.append((OP_COPY, None, 0, [n], fresh))
        return nodes, edges + copies, list(self.sources), targets

    def compile(self, lib):
        """Lower to a cg_term owned by `lib` (cached per library)."""
        key = lib._path
        if key in self._compiled:
            return self._compiled[key]
        nodes, edges, sources, targets = self.lowered()
        t = C.c_void_p()
        _chk(lib, lib.cg_term_create(C.byref(t)))
        handle = _TermHandle(lib, t)
        nid = C.c_uint32()
        for label in nodes:
            _chk(lib, lib.cg_term_add_node(t, label, C.byref(nid)))
        for op, p, scalar, src, tgt in edges:
            s = (C.c_uint32 * builtins.max(len(src), 1))(*src)
            g = (C.c_uint32 * builtins.max(len(tgt), 1))(*tgt)
            _chk(lib, lib.cg_term_add_op(t, op, p.encode() if p is not None else None, scalar,
                                         s, len(src), g, len(tgt), None))
        s = (C.c_uint32 * builtins.max(len(sources), 1))(*sources)
        g = (C.c_uint32 * builtins.max(len(targets), 1))(*targets)
        _chk(lib, lib.cg_term_set_boundary(t, s, len(sources), g, len(targets)))
        self._compiled[key] = handle
        return handle

    def stats(self, lib):
        h = self.compile(lib)
        a, b = C.c_size_t(), C.c_size_t()
        st = lib.cg_term_stats(h.ptr, C.byref(a), C.byref(b))
        if st:
            raise abi.InterpreterError(st, lib.cg_interp_last_error().decode(), 0)
        return {"ops": a.value, "layers": b.value}


class _TermHandle:
    def __init__(self, lib, ptr):
        self.lib, self.ptr = lib, ptr

    def __del__(self):
        if self.ptr:
            self.lib.cg_term_destroy(self.ptr)
            self.ptr = None


def _chk(lib, st):
    if st:
        raise abi.InterpreterError(st, lib.cg_interp_last_error().decode(), 0)


def build_typed(source_labels, f):
    """crate::util::build_typed: run `f(builder, source vars)` and close the term."""
    b = Builder()
    args = [Var(b, b.new_node(l), l) for l in source_labels]
    results = f(b, args)
    return Term(b, args, list(results))


# ---------------------------------------------------------------------------------------------
# lang/ops.rs

def pow(builder, value, exponent):  # noqa: A001
    return builder.fn_operation([value, exponent], TENSOR, OP_POW)


def sin(builder, value):
    return builder.fn_operation([value], TENSOR, OP_SIN)


def cos(builder, value):
    return builder.fn_operation([value], TENSOR, OP_COS)


def param(builder, p):
    """lang/ops.rs:94-101 plus stdlib to_load_ops: a Load of the parameter named `p`."""
    return builder.fn_operation([], TENSOR, OP_LOAD, path=p)


def lit(builder, x):
    """lang/ops.rs:103-110 and stdlib/ops.rs:52-54 (`Into<Literal>`: f32 -> F32, u32 via nat())."""
    if isinstance(x, NatLit):
        return builder.fn_operation([], NAT, OP_NAT_CONST, scalar=int(x))
    if isinstance(x, U32Lit):
        return builder.fn_operation([], TENSOR, OP_SCALAR_U32, scalar=int(x))
    bits = struct.unpack("<I", struct.pack("<f", float(x)))[0]
    return builder.fn_operation([], TENSOR, OP_SCALAR_F32, scalar=bits)


def pack(builder, extents):
    for x in extents:
        assert x.label == NAT
    return builder.fn_operation(list(extents), SHAPE, OP_PACK)


def unpack(builder, n, x):
    """unpack::<N>(builder, x)"""
    assert x.label == SHAPE, "input to unpack was not a shape"
    return builder.operation([x], [NAT] * n, OP_UNPACK)


def shape(builder, x):
    return builder.fn_operation([x], SHAPE, OP_SHAPE)


def dtype_constant(builder, d):
    return builder.fn_operation([], DTYPE, OP_DTYPE_CONST, scalar=int(d))


def broadcast(builder, x, s):
    return builder.fn_operation([x, s], TENSOR, OP_BROADCAST)


expand = broadcast


def reshape(builder, t, x):
    return builder.fn_operation([t, x], TENSOR, OP_RESHAPE)


def max(builder, x):  # noqa: A001
    return builder.fn_operation([x], TENSOR, OP_MAX)


def sum(builder, x):  # noqa: A001
    return builder.fn_operation([x], TENSOR, OP_SUM)


def argmax(builder, x):
    return builder.fn_operation([x], TENSOR, OP_ARGMAX)


def nat_to_u32(builder, n):
    return builder.fn_operation([n], TENSOR, OP_NAT_TO_U32)


def lt(builder, x, y):
    return builder.fn_operation([x, y], TENSOR, OP_LT)


def eq(builder, x, y):
    return builder.fn_operation([x, y], TENSOR, OP_EQ)


def matmul(builder, f, g):
    assert f.label == TENSOR and g.label == TENSOR
    return builder.fn_operation([f, g], TENSOR, OP_MATMUL)


def dtype(builder, x):
    assert x.label == TENSOR
    return builder.fn_operation([x], DTYPE, OP_DTYPE)


# ---------------------------------------------------------------------------------------------
# stdlib/ops.rs: wrappers taking `impl IntoNatVar` / `impl IntoDtypeVar`

def to_nat(builder, x):
    """IntoNatVar (stdlib/ops.rs:83-113): a Var stays, an integer becomes a Nat literal."""
    if isinstance(x, Var):
        return x
    return lit(builder, nat(int(x)))


def to_dtype(builder, d):
    """IntoDtypeVar (stdlib/ops.rs:115-129).  The reference's impl for `Dtype` ignores its
    argument and always emits F32; every call site passes F32, and so must callers here."""
    if isinstance(d, Var):
        return d
    return dtype_constant(builder, abi.F32)


def cast(builder, x, d):
    dv = to_dtype(builder, d)
    assert x.label == TENSOR and dv.label == DTYPE
    return builder.fn_operation([x, dv], TENSOR, OP_CAST)


def arange(builder, end):
    return builder.fn_operation([to_nat(builder, end)], TENSOR, OP_ARANGE)


def concat(builder, dim, x, y):
    return builder.fn_operation([x, y, to_nat(builder, dim)], TENSOR, OP_CONCAT)


def topk(builder, k, x):
    kv = to_nat(builder, k)
    assert kv.label == NAT and x.label == TENSOR
    values, indices = builder.operation([x, kv], [TENSOR, TENSOR], OP_TOPK)
    return values, indices


def index(builder, dim, idx, x):
    return builder.fn_operation([x, to_nat(builder, dim), idx], TENSOR, OP_INDEX)


def slice(builder, dim, start, len, x):  # noqa: A001,A002
    return builder.fn_operation(
        [x, to_nat(builder, dim), to_nat(builder, start), to_nat(builder, len)], TENSOR, OP_SLICE)


def get(builder, dim, start, x):
    return slice(builder, dim, start, 1, x)


def constant(builder, x, s):
    """stdlib/ops.rs:61-64: a literal broadcast to shape `s`."""
    return broadcast(builder, lit(builder, x), s)


def inverse(builder, x):
    sh = shape(builder, x)
    one = constant(builder, 1.0, sh)
    return one / x


def transpose(builder, a, b, x):
    return builder.fn_operation([x, to_nat(builder, a), to_nat(builder, b)], TENSOR, OP_TRANSPOSE)


def make_shape(builder, *dims):
    """the shape! macro: pack Nat vars and integer literals into a shape."""
    return pack(builder, [to_nat(builder, d) for d in dims])


# ---------------------------------------------------------------------------------------------
# stdlib/module.rs

class Module:
    """trait Module<A, B>: `path`, `sort` (object labels of sources and targets) and `def_`."""

    def path(self):
        raise NotImplementedError

    def sort(self):
        """([source labels], [target labels])"""
        raise NotImplementedError

    def def_(self, builder, args):
        raise NotImplementedError

    def inline(self, builder, args):
        return self.def_(builder, args)

    def op(self, builder, args):
        """One Definition edge named `self.path()` (module.rs:44-55)."""
        return builder.operation(list(args), self.sort()[1], OP_DEF, path=self.path())

    def call(self, builder, args):
        (r,) = self.op(builder, args)
        return r

    def term(self):
        src, tgt = self.sort()
        t = build_typed(src, lambda b, a: self.inline(b, a))
        got = [t.builder.nodes[n] for n in t.targets]
        assert got == list(tgt), "definition returned vars of other sorts than declared"
        return t

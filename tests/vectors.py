"""Checks shared by the CPU (oracle) and GPU (HIP) suites: the reference's own test vectors
(tests/golden/reference_vectors.json) replayed on whichever backend is handed in."""
import importlib
import json
import os

import numpy as np

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))

cg = importlib.import_module("catgrad-rs_amd")
lang, nn = cg.lang, cg.nn
helpers = importlib.import_module("catgrad-rs_amd.llm.helpers")
T = lang.TENSOR


def f32(x):
    return np.asarray(x, dtype=np.float32)


def u32(x):
    return np.asarray(x, dtype=np.uint32)


def approx6(a):
    """NdArray::approx(6) of the legacy tests: round(x * 1e6) / 1e6 in f32."""
    b = np.float32(10.0) ** 6
    return np.round(f32(a) * b) / b


class Fn(lang.Module):
    """A throw-away Module around a Python function of Vars."""

    def __init__(self, name, n_in, n_out, fn):
        self.name, self.n_in, self.n_out, self.fn = name, n_in, n_out, fn

    def path(self):
        return lang.path(["test", self.name])

    def sort(self):
        return [T] * self.n_in, [T] * self.n_out

    def def_(self, builder, args):
        r = self.fn(builder, *args)
        return list(r) if isinstance(r, (list, tuple)) else [r]


def run(be, fn, n_out, *arrays, params=None):
    """Build a term from `fn`, run it through the native evaluator on `be`."""
    P = cg.Parameters()
    for k, v in (params or {}).items():
        P[k] = be.tensor(v)
    it = cg.Interpreter(be, cg.stdlib(), P)
    term = Fn("f", len(arrays), n_out, fn).term()
    outs = it.run(term, [be.tensor(a) for a in arrays])
    return [be.numpy(o) for o in outs]


def check_backend_unit_vectors(be):
    """ndarray.rs:630-821 and the legacy evaluator/kernel vectors, straight on the Backend."""
    g = GOLDEN["ndarray_batched_matmul"]
    out = be.numpy(be.matmul(be.tensor(f32(g["lhs"]), g["lhs_shape"]), be.tensor(f32(g["rhs"]), g["rhs_shape"])))
    assert out.shape == tuple(g["shape"]) and np.array_equal(out.ravel(), f32(g["expected"]))
    for name, op in (("ndarray_add", be.add), ("ndarray_sub", be.sub)):
        g = GOLDEN[name]
        out = be.numpy(op(be.tensor(f32(g["x"]), g["shape"]), be.tensor(f32(g["y"]), g["shape"])))
        assert np.array_equal(out.ravel(), f32(g["expected"]))
    for name, op, cast in (("ndarray_sum_u32", be.sum, u32), ("ndarray_sum_f32", be.sum, f32),
                           ("ndarray_max_f32", be.max, f32), ("ndarray_max_u32", be.max, u32),
                           ("ndarray_max_f32_3d", be.max, f32)):
        g = GOLDEN[name]
        out = be.numpy(op(be.tensor(cast(g["x"]), g["shape"])))
        assert out.shape == tuple(g["out_shape"]), name
        assert np.array_equal(out.ravel(), cast(g["expected"])), name
    g = GOLDEN["legacy_sin_cos"]
    x = be.tensor(f32(g["x"]), (2, 2))
    assert np.allclose(be.to_vec(be.sin(x)), f32(g["sin"]), atol=2e-6)
    assert np.allclose(be.to_vec(be.cos(x)), f32(g["cos"]), atol=2e-6)
    g = GOLDEN["legacy_pow"]
    out = be.to_vec(be.pow(be.tensor(f32(g["x"]), (2, 2)), be.tensor(f32(g["y"]), (2, 2))))
    assert np.allclose(out, f32(g["expected"]), rtol=1e-6)
    out = be.to_vec(be.pow(be.tensor(u32(g["x"]), (2, 2)), be.tensor(u32(g["y"]), (2, 2))))
    assert np.array_equal(out, u32(g["expected"]))
    g = GOLDEN["legacy_lt"]
    out = be.to_vec(be.lt(be.tensor(f32(g["x"]), (2, 3)), be.tensor(f32(g["y"]), (2, 3))))
    assert np.array_equal(out, f32(g["expected"]))
    g = GOLDEN["legacy_matmul_transposed"]
    mt = be.transpose(be.tensor(f32(g["mt"]), g["mt_shape"]), 0, 1)      # strides [1, 2]
    out = be.to_vec(be.matmul(be.tensor(f32(g["x"]), g["x_shape"]), mt))
    assert np.array_equal(out, f32(g["expected"]))
    g = GOLDEN["legacy_max"]
    assert np.array_equal(be.to_vec(be.max(be.tensor(f32(g["x"]), g["shape"]))), f32(g["expected"]))
    g = GOLDEN["legacy_argmax"]
    assert np.array_equal(be.to_vec(be.argmax(be.tensor(f32(g["x"]), g["shape"]))), u32(g["expected"]))
    g = GOLDEN["legacy_sum"]
    assert np.array_equal(be.to_vec(be.sum(be.tensor(f32(g["x"]), g["shape"]))), f32(g["expected"]))
    g = GOLDEN["legacy_topk"]
    v, i = be.topk(be.tensor(f32(g["x"]), g["shape"]), g["k"])
    assert np.array_equal(be.to_vec(v), f32(g["values"])) and np.array_equal(be.to_vec(i), u32(g["indices"]))
    g = GOLDEN["legacy_gemm"]
    out = be.to_vec(be.matmul(be.tensor(f32(g["a"]), g["a_shape"]), be.tensor(f32(g["b"]), g["b_shape"])))
    assert np.array_equal(out, f32(g["c"]))
    out = be.to_vec(be.matmul(be.tensor(f32(g["f"]), g["f_shape"]), be.tensor(f32(g["g"]), g["g_shape"])))
    assert np.array_equal(out, f32(g["h"]))


def check_interpreter_vectors(be):
    """catgrad/tests/test_interpreter.rs:51-191 replayed through the evaluator."""
    g = GOLDEN["interp_add_u32"]
    x = u32(g["x"]).reshape(g["shape"])
    (out,) = run(be, lambda b, p, q: p + q, 1, x, x)
    exp = be.tensor(u32(g["expected"]), g["shape"])
    assert be.compare(be.tensor(out), exp)

    g = GOLDEN["interp_batch_matmul"]
    (out,) = run(be, lang.matmul, 1, f32(g["x0"]).reshape(g["x0_shape"]), f32(g["x1"]).reshape(g["x1_shape"]))
    assert out.shape == tuple(g["shape"]) and np.array_equal(out.ravel(), f32(g["expected"]))

    g = GOLDEN["interp_exp"]
    x = f32(g["x"]).reshape(g["shape"])
    it = cg.Interpreter(be, cg.stdlib())
    (y,) = it.run(nn.Exp().term(), [be.tensor(x)])
    got, exp = be.to_vec(y), np.exp(x.ravel())           # f32::exp
    assert np.all(np.abs(got - exp) <= g["atol"] + g["rtol"] * np.abs(exp))

    g = GOLDEN["interp_topk"]
    v, i = run(be, lambda b, x: lang.topk(b, g["k"], x), 2, f32(g["x"]).reshape(g["shape"]))
    assert np.array_equal(v.ravel(), f32(g["values"])) and np.array_equal(i.ravel(), u32(g["indices"]))
    assert i.dtype == np.uint32


def check_nn_vectors(be):
    """legacy/nn/layers.rs:735-877, 1192-1208 through the Interpreter-path stdlib definitions."""
    g = GOLDEN["legacy_activations"]
    x = f32(g["x"]).reshape(1, 3)
    it = cg.Interpreter(be, cg.stdlib())
    for name, mod in (("tanh", nn.Tanh()), ("gelu", nn.Gelu()), ("sigmoid", nn.Sigmoid()),
                      ("silu", nn.Silu()), ("softmax", nn.Softmax())):
        # as a Definition op (handle_definition) ...
        (y,) = run(be, lambda b, v, m=mod: m.call(b, [v]), 1, x)
        assert np.array_equal(approx6(y.ravel()), f32(g[name])), name
        # ... and evaluated directly
        (y2,) = it.run(mod.term(), [be.tensor(x)])
        assert np.array_equal(approx6(be.to_vec(y2)), f32(g[name])), name
    g = GOLDEN["legacy_softmax_offset"]
    (y,) = run(be, nn.softmax, 1, f32(g["x"]).reshape(1, 3))
    assert np.array_equal(approx6(y.ravel()), f32(g["expected"]))
    g = GOLDEN["legacy_rmsnorm_raw"]
    (y,) = run(be, lambda b, v: helpers.rmsnorm_raw(b, g["eps"], v), 1, f32(g["x"]).reshape(1, 1, 5))
    assert np.array_equal(approx6(y.ravel()), f32(g["expected"]))
    g = GOLDEN["legacy_layernorm_raw"]
    (y,) = run(be, lambda b, v: helpers.layernorm_raw(b, g["eps"], v), 1, f32(g["x"]).reshape(1, 1, 5))
    assert np.allclose(y.ravel(), f32(g["expected"]), atol=1.5e-6)
    g = GOLDEN["legacy_linear"]
    x = f32(g["x"]).reshape([1] + g["x_shape"])
    params = {"l.weight": f32(g["w"]).reshape(g["w_shape"]), "l.bias": f32(g["b"])}
    (y,) = run(be, lambda b, v: nn.linear(b, 3, 2, lang.path(["l"]), v), 1, x, params=params)
    assert np.array_equal(approx6(y.ravel()), f32(g["with_bias"]))
    (y,) = run(be, lambda b, v: nn.linear_no_bias(b, 3, 2, lang.path(["l"]), v), 1, x, params=params)
    assert np.array_equal(approx6(y.ravel()), f32(g["no_bias"]))
    g = GOLDEN["legacy_causal_mask"]

    def mask(b, v):  # size taken from the input's shape, as the models do
        (n,) = lang.unpack(b, 1, lang.shape(b, v))
        return helpers.causal_mask(b, n)
    (m,) = run(be, mask, 1, np.zeros(g["size"], np.float32))
    fmin = np.finfo(np.float32).min
    assert m.shape == (3, 3)
    assert np.array_equal(m.ravel(), f32(g["pattern"]) * fmin)       # 0 * MIN = -0.0 == 0


def _points(a, pts, what):
    for idx, v in pts:
        assert a[tuple(idx)] == v, (what, idx, float(a[tuple(idx)]), v)


def check_legacy_shape_vectors(be):
    """The shape-op vectors of catgrad-llm/src/legacy/nn/layers.rs (repeat_kv, index, narrow, concat,
    transpose + reshape, expand, arange, cast, batched linear), on the Backend methods they map to; the
    reference asserts single elements (`get(&[..])`), so single elements are what is compared."""
    def arange_f32(n):
        return be.cast(be.arange(n), cg.abi.F32)
    g = GOLDEN["legacy_repeat_kv"]
    x = np.arange(g["x_arange"], dtype=np.float32).reshape(g["x_shape"])
    (y,) = run(be, lambda b, v: helpers.repeat_kv(b, g["rep"], v), 1, x)
    assert list(y.shape) == g["shape"]
    _points(y, g["points"], "repeat_kv")
    g = GOLDEN["legacy_index"]
    x = be.broadcast(arange_f32(g["x_arange"]), g["x_expand"])
    for c in g["cases"]:
        y = be.numpy(be.index(x, c["dim"], be.tensor(u32(c["indices"]))))
        assert list(y.shape) == c["shape"]
        _points(y, c["points"], "index")
    g = GOLDEN["legacy_narrow"]
    x = be.reshape(arange_f32(g["x_arange"]), g["x_shape"])
    for c in g["cases"]:
        y = be.numpy(be.slice(x, c["dim"], c["start"], c["len"]))
        assert list(y.shape) == c["shape"]
        _points(y, c["points"], "narrow")
    g = GOLDEN["legacy_concat"]
    a, b_ = be.tensor(f32(g["x"]), g["shape"]), be.tensor(f32(g["y"]), g["shape"])
    for dim in (0, 1):
        y = be.numpy(be.concat(a, b_, dim))
        assert list(y.shape) == g[f"dim{dim}_shape"] and np.array_equal(y.ravel(), f32(g[f"dim{dim}"]))
    g = GOLDEN["legacy_transpose_reshape"]
    b_ = be.reshape(arange_f32(g["x_arange"]), g["b_shape"])
    assert np.array_equal(be.to_vec(b_), f32(g["b"]))
    d = be.reshape(be.transpose(b_, 0, 1), g["d_shape"])   # a reshape of a transposed view reorders
    m = be.numpy(be.matmul(d, b_))
    assert list(m.shape) == g["m_shape"] and np.array_equal(m.ravel(), f32(g["m"]))
    g = GOLDEN["legacy_expand"]
    y = be.numpy(be.broadcast(arange_f32(g["x_arange"]), g["shape"]))
    assert list(y.shape) == g["shape"]
    _points(y, g["points"], "expand")
    g = GOLDEN["legacy_arange_expand_reshape"]
    e = be.broadcast(arange_f32(g["x_arange"]), g["expand"])
    _points(be.numpy(e), g["e_points"], "arange/expand")
    r = be.numpy(be.reshape(e, g["reshape"]))
    assert list(r.shape) == g["reshape"]
    _points(r, g["r_points"], "arange/reshape")
    g = GOLDEN["legacy_cast"]
    i = be.arange(g["n"])
    assert np.array_equal(be.to_vec(be.cast(i, cg.abi.F32)), f32(g["int_to_f32"]))
    assert np.array_equal(be.to_vec(be.cast(be.cast(i, cg.abi.F32), cg.abi.U32)), u32(g["f32_to_int"]))
    g = GOLDEN["legacy_linear_batch"]
    x = np.broadcast_to(f32(g["x"]).reshape(g["x_shape"]), [g["batch"]] + g["x_shape"]).copy()
    params = {"l.weight": f32(g["w"]).reshape(g["w_shape"]), "l.bias": f32(g["b"])}

    def batched_linear(b, v):  # the batch folded into the rows and back: the batch-correct reading of nn.linear
        qm = importlib.import_module("catgrad-rs_amd.llm.qwen_moe")
        f, bb, s = qm.fold_batch(b, v)
        return qm.unfold_batch(b, bb, s, nn.linear(b, 3, 2, lang.path(["l"]), f))
    (y,) = run(be, batched_linear, 1, x, params=params)
    assert y.shape == (2, 2, 2) and np.array_equal(approx6(y.ravel()), f32(g["expected"]))


def bf16_round(a):
    """f32 array rounded to the nearest bf16 (ties to even), as f32."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)

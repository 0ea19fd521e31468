"""Pins the CPU oracle (oracle/ndarray_oracle.cpp): the reference's own test vectors, then what
the mathematics fixes for the functions no reference test covers."""
import numpy as np
import pytest

import vectors


def test_reference_backend_vectors(oracle):
    vectors.check_backend_unit_vectors(oracle)


def test_reference_interpreter_vectors(oracle):
    vectors.check_interpreter_vectors(oracle)


def test_reference_nn_vectors(oracle):
    vectors.check_nn_vectors(oracle)


def test_reference_legacy_shape_vectors(oracle):
    vectors.check_legacy_shape_vectors(oracle)


def bf(x):
    return np.asarray(x, np.float32)


def test_elementwise_is_ieee(oracle):
    """+ - * / neg lt eq are fixed by IEEE-754: numpy float32 is an independent statement."""
    g = np.random.default_rng(1)
    a = g.standard_normal((37, 13)).astype(np.float32) * 100
    b = g.standard_normal((37, 13)).astype(np.float32)
    b[0, 0] = 0
    ta, tb = oracle.tensor(a), oracle.tensor(b)
    with np.errstate(all="ignore"):
        for name, ref in (("add", a + b), ("sub", a - b), ("mul", a * b), ("div", a / b),
                          ("lt", (a < b).astype(np.float32)), ("eq", (a == b).astype(np.float32))):
            out = oracle.numpy(getattr(oracle, name)(ta, tb))
            assert np.array_equal(out.view(np.uint32), ref.astype(np.float32).view(np.uint32)), name
    assert np.array_equal(oracle.numpy(oracle.neg(ta)), -a)


def test_u32_wrapping_semantics(cg, oracle):
    a = np.array([0xFFFFFFFF, 5, 0x80000000, 7], np.uint32)
    b = np.array([2, 7, 2, 0], np.uint32)
    ta, tb = oracle.tensor(a), oracle.tensor(b)
    assert list(oracle.to_vec(oracle.add(ta, tb))) == [1, 12, 0x80000002, 7]
    assert list(oracle.to_vec(oracle.sub(tb, ta))) == [3, 2, 0x80000002, 0xFFFFFFF9]
    assert list(oracle.to_vec(oracle.mul(ta, tb))) == [0xFFFFFFFE, 35, 0, 0]
    assert list(oracle.to_vec(oracle.pow(ta, tb))) == [1, 78125, 0, 1]
    assert list(oracle.to_vec(oracle.neg(ta))) == [1, 0xFFFFFFFB, 0x80000000, 0xFFFFFFF9]
    with pytest.raises(cg.BackendPanic, match="divide by zero"):
        oracle.div(ta, tb)


def test_pow_sin_cos_against_f64(oracle):
    g = np.random.default_rng(2)
    a = np.abs(g.standard_normal(500)).astype(np.float32) * 5 + 0.01
    b = (g.standard_normal(500) * 3).astype(np.float32)
    got = oracle.to_vec(oracle.pow(oracle.tensor(a), oracle.tensor(b)))
    assert np.allclose(got, np.power(a.astype(np.float64), b.astype(np.float64)), rtol=3e-7)
    x = (g.standard_normal(500) * 100).astype(np.float32)
    assert np.allclose(oracle.to_vec(oracle.sin(oracle.tensor(x))), np.sin(x.astype(np.float64)), atol=1e-7)
    assert np.allclose(oracle.to_vec(oracle.cos(oracle.tensor(x))), np.cos(x.astype(np.float64)), atol=1e-7)
    # the masked-softmax case: a hugely negative exponent gives exactly 0, never NaN
    e = oracle.tensor(bf([2.7182817, 2.7182817]))
    y = oracle.tensor(bf([-3.4028235e38, -200.0]))
    assert list(oracle.to_vec(oracle.pow(e, y))) == [0.0, 0.0]


def test_cast_is_rust_as(cg, oracle):
    a = bf([0.0, -0.0, 0.9, 1.5, -1.5, 4294967040.0, 4294967296.0, 1e20, -1e20, np.inf, -np.inf, np.nan])
    got = oracle.to_vec(oracle.cast(oracle.tensor(a), cg.U32))
    assert list(got) == [0, 0, 0, 1, 0, 4294967040, 4294967295, 4294967295, 0, 4294967295, 0, 0]
    u = np.array([0, 1, 16777217, 2**31 + 129, 2**32 - 1], np.uint32)
    got = oracle.to_vec(oracle.cast(oracle.tensor(u), cg.F32))
    assert np.array_equal(got, u.astype(np.float32))
    t = oracle.tensor(u)
    assert oracle.cast(t, cg.U32).ptr == t.ptr          # same dtype: the value itself


def test_shape_ops_against_numpy(oracle):
    g = np.random.default_rng(3)
    a = g.standard_normal((3, 4, 5)).astype(np.float32)
    t = oracle.tensor(a)
    assert np.array_equal(oracle.numpy(oracle.transpose(t, 0, 2)), a.transpose(2, 1, 0))
    assert np.array_equal(oracle.numpy(oracle.transpose(oracle.transpose(t, 0, 2), 0, 2)), a)
    assert np.array_equal(oracle.numpy(oracle.reshape(oracle.transpose(t, 1, 2), (15, 4))),
                          a.transpose(0, 2, 1).reshape(15, 4))
    assert np.array_equal(oracle.numpy(oracle.slice(t, 1, 1, 2)), a[:, 1:3])
    assert np.array_equal(oracle.numpy(oracle.broadcast(oracle.tensor(a[:, :1]), (2, 3, 4, 5))),
                          np.broadcast_to(a[:, :1], (2, 3, 4, 5)))
    b = g.standard_normal((3, 2, 5)).astype(np.float32)
    c = oracle.concat(t, oracle.tensor(b), 1)
    assert np.array_equal(oracle.numpy(c), np.concatenate([a, b], 1))
    assert np.array_equal(oracle.numpy(oracle.slice(c, 1, 4, 2)), b)       # concat then slice
    idx = np.array([[2], [0], [2]], np.uint32)                              # any rank: flattened
    assert np.array_equal(oracle.numpy(oracle.index(t, 0, oracle.tensor(idx))), a[[2, 0, 2]])
    assert np.array_equal(oracle.numpy(oracle.index(t, 2, oracle.arange(5))), a)
    assert np.array_equal(oracle.to_vec(oracle.arange(6)), np.arange(6, dtype=np.uint32))
    assert oracle.arange(0).shape == (0,)


def test_total_order_rules_brute_force(oracle):
    """argmax = last maximum under total_cmp; topk = stable descending sort; max ignores NaN and
    floors at f32::MIN.  Checked against a pure-Python statement of f32::total_cmp."""
    specials = bf([np.nan, -np.nan, np.inf, -np.inf, 0.0, -0.0, 1.0, -1.0, 1.0, 3.5, 3.5])
    specials[1] = np.frombuffer(np.uint32(0xFFC00000).tobytes(), np.float32)[0]

    def key(v):
        b = int(np.float32(v).view(np.int32))
        return b ^ (((b >> 31) & 0xFFFFFFFF) >> 1)

    g = np.random.default_rng(4)
    for _ in range(200):
        row = g.choice(specials, size=7)
        t = oracle.tensor(row.reshape(1, 7))
        keys = [key(v) for v in row]
        best = max(range(7), key=lambda i: (keys[i], i))
        assert oracle.to_vec(oracle.argmax(t))[0] == best
        order = sorted(range(7), key=lambda i: (-keys[i], i))
        v, ix = oracle.topk(t, 4)
        assert list(oracle.to_vec(ix)) == order[:4]
        assert np.array_equal(oracle.to_vec(v).view(np.uint32), row[order[:4]].view(np.uint32))
        finite = [x for x in row if not np.isnan(x)]
        exp = max([np.finfo(np.float32).min] + finite)
        assert oracle.to_vec(oracle.max(t))[0] == np.float32(exp)
    u = np.array([[3, 9, 9, 1]], np.uint32)
    assert oracle.to_vec(oracle.argmax(oracle.tensor(u)))[0] == 2


def test_sum_matmul_against_f64(oracle):
    g = np.random.default_rng(5)
    a = g.standard_normal((6, 1000)).astype(np.float32)
    s = oracle.numpy(oracle.sum(oracle.tensor(a)))
    assert s.shape == (6, 1)
    assert np.allclose(s.ravel(), a.astype(np.float64).sum(1), rtol=0, atol=1e-4 * np.abs(a).sum(1).max())
    for (m, k, n) in [(1, 7, 3), (13, 300, 37), (6, 256, 16), (70, 513, 33)]:
        x = g.standard_normal((2, m, k)).astype(np.float32)
        y = g.standard_normal((2, k, n)).astype(np.float32)
        out = oracle.numpy(oracle.matmul(oracle.tensor(x), oracle.tensor(y)))
        ref = np.matmul(x.astype(np.float64), y.astype(np.float64))
        scale = np.matmul(np.abs(x).astype(np.float64), np.abs(y).astype(np.float64))
        assert np.all(np.abs(out - ref) <= 1e-5 * scale)
    # identity and linearity
    eye = np.eye(9, dtype=np.float32)
    z = g.standard_normal((9, 9)).astype(np.float32)
    assert np.array_equal(oracle.numpy(oracle.matmul(oracle.tensor(z), oracle.tensor(eye))), z)


def test_softmax_rmsnorm_invariants(oracle):
    g = np.random.default_rng(6)
    x = g.standard_normal((1, 5, 33)).astype(np.float32) * 4
    (p,) = vectors.run(oracle, vectors.nn.softmax, 1, x)
    assert np.allclose(p.sum(-1), 1, atol=1e-5) and np.all(p >= 0)
    (p2,) = vectors.run(oracle, vectors.nn.softmax, 1, x + np.float32(3.0))
    assert np.allclose(p, p2, atol=1e-5)                                    # shift invariance
    ref = np.exp(x.astype(np.float64) - x.max(-1, keepdims=True))
    assert np.allclose(p, ref / ref.sum(-1, keepdims=True), atol=1e-6)
    (r,) = vectors.run(oracle, lambda b, v: vectors.helpers.rmsnorm_raw(b, 0.0, v), 1, x)
    assert np.allclose(np.sqrt((r.astype(np.float64) ** 2).mean(-1)), 1, atol=1e-5)  # unit RMS

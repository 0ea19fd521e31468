"""HIP backend vs the CPU oracle, op by op, through the C ABI, on the same seeded inputs.

Bar: bit-exact for shape / index / argmax / gather / comparison / integer ops and for the IEEE
basic operations; rel 1e-4 for f32 transcendental, sum and matmul; rel 2e-2 in bf16 mode.
"""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL_F32 = 1e-4
RTOL_BF16 = 2e-2


def rng(seed):
    if not isinstance(seed, int):
        seed = zlib.crc32(repr(seed).encode())
    return np.random.default_rng(seed)


def both(oracle, hip, fn, *arrays):
    """Run fn(backend, *tensors) on both backends; return the two numpy results."""
    outs = []
    for be in (oracle, hip):
        ts = [be.tensor(a) for a in arrays]
        r = fn(be, *ts)
        rs = r if isinstance(r, tuple) else (r,)
        outs.append([be.numpy(t) for t in rs])
    return outs


def assert_bits(a, b):
    assert a.shape == b.shape and a.dtype == b.dtype
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), \
        f"bit mismatch: {np.flatnonzero(a.view(np.uint32).ravel() != b.view(np.uint32).ravel())[:8]}"


def assert_close(ref, got, rtol, scale=None):
    assert ref.shape == got.shape
    scale = np.abs(ref) if scale is None else scale
    err = np.abs(ref.astype(np.float64) - got.astype(np.float64))
    finite = np.isfinite(ref)
    assert np.array_equal(np.isnan(ref), np.isnan(got))
    assert np.array_equal(ref[~finite & ~np.isnan(ref)], got[~finite & ~np.isnan(ref)])
    bad = err[finite] > rtol * scale[finite] + 1e-30
    assert not bad.any(), f"max rel err {np.max(err[finite] / (scale[finite] + 1e-30))}"


@pytest.fixture(params=["lazy", "eager", "nopat"])
def dev(request, hip, hip_eager, hip_nopat):
    return {"lazy": hip, "eager": hip_eager, "nopat": hip_nopat}[request.param]


SHAPES = [(7,), (4, 4), (3, 5, 8), (2, 3, 4, 5), (1, 1), (257, 3), (64, 128)]


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "lt", "eq"])
@pytest.mark.parametrize("shape", SHAPES)
def test_binary_f32_bit_exact(oracle, dev, op, shape):
    g = rng((op, shape))
    a = g.standard_normal(shape).astype(np.float32)
    b = g.standard_normal(shape).astype(np.float32)
    b.ravel()[::3] = a.ravel()[::3]          # some equal pairs for lt/eq
    a.ravel()[:1] = np.float32(np.inf)
    if a.size > 2:
        b.ravel()[1] = np.float32(0.0)
        a.ravel()[2] = np.float32(np.nan)
    r, d = both(oracle, dev, lambda be, x, y: getattr(be, op)(x, y), a, b)
    # IEEE basic operations and comparisons are exactly specified
    nan = np.isnan(r[0])
    assert np.array_equal(nan, np.isnan(d[0]))
    assert_bits(np.where(nan, 0, r[0]).astype(np.float32), np.where(nan, 0, d[0]).astype(np.float32))


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "pow", "lt", "eq"])
@pytest.mark.parametrize("shape", SHAPES[:4])
def test_binary_u32_bit_exact(oracle, dev, op, shape):
    g = rng((op, shape, "u"))
    a = g.integers(0, 2**32, shape, dtype=np.uint64).astype(np.uint32)
    b = g.integers(1, 2**32, shape, dtype=np.uint64).astype(np.uint32)
    if op == "pow":
        b = (b % 40).astype(np.uint32)
    if op in ("lt", "eq"):
        b.ravel()[::2] = a.ravel()[::2]
    r, d = both(oracle, dev, lambda be, x, y: getattr(be, op)(x, y), a, b)
    assert_bits(r[0], d[0])


def test_pow_f32(oracle, dev):
    g = rng(5)
    a = np.abs(g.standard_normal((33, 17))).astype(np.float32) * 3
    b = (g.standard_normal((33, 17)) * 4).astype(np.float32)
    a[0, :6] = [0.0, -1.0, -2.0, np.inf, 2.7182817, 1.0]
    b[0, :6] = [0.0, 2.0, 0.5, -1.0, -3.4e38, np.nan]
    r, d = both(oracle, dev, lambda be, x, y: be.pow(x, y), a, b)
    assert_close(r[0], d[0], RTOL_F32)


@pytest.mark.parametrize("op", ["sin", "cos", "neg"])
def test_unary_f32(oracle, dev, op):
    a = (rng(6).standard_normal((19, 40)) * 50).astype(np.float32)
    r, d = both(oracle, dev, lambda be, x: getattr(be, op)(x), a)
    if op == "neg":
        assert_bits(r[0], d[0])
    else:
        assert_close(r[0], d[0], RTOL_F32, scale=np.ones_like(r[0]))


def test_neg_u32_and_sin_u32_rejected(cg, oracle, dev):
    a = np.array([0, 1, 2**31, 2**32 - 1], dtype=np.uint32)
    r, d = both(oracle, dev, lambda be, x: be.neg(x), a)
    assert_bits(r[0], d[0])
    for be in (oracle, dev):
        with pytest.raises(cg.BackendPanic):
            be.sin(be.tensor(a))
        with pytest.raises(cg.BackendPanic):
            be.cos(be.tensor(a))


def test_cast_rust_as_semantics(cg, oracle, dev):
    a = np.array([0.0, -0.0, 0.9, 1.5, -1.5, 4294967040.0, 4294967296.0, 1e20, -1e20, np.inf,
                  -np.inf, np.nan, 16777217.0, 2.5], dtype=np.float32)
    r, d = both(oracle, dev, lambda be, x: be.cast(x, cg.U32), a)
    assert_bits(r[0], d[0])
    assert list(r[0][:12]) == [0, 0, 0, 1, 0, 4294967040, 4294967295, 4294967295, 0, 4294967295, 0, 0]
    u = np.array([0, 1, 16777217, 2**31 + 129, 2**32 - 1], dtype=np.uint32)
    r, d = both(oracle, dev, lambda be, x: be.cast(x, cg.F32), u)
    assert_bits(r[0], d[0])
    assert_bits(r[0], u.astype(np.float32))
    # same dtype: identity
    r, d = both(oracle, dev, lambda be, x: be.cast(x, cg.U32), u)
    assert_bits(r[0], d[0])


def test_shape_mismatch_panics(cg, oracle, dev):
    for be in (oracle, dev):
        x = be.tensor(np.zeros((2, 3), np.float32))
        y = be.tensor(np.zeros((3, 2), np.float32))
        with pytest.raises(cg.ShapeError, match="Shape mismatch in operation"):
            be.add(x, y)
        with pytest.raises(cg.ShapeError):
            be.ndarray_from_vec_f32(np.zeros(5, np.float32), (2, 3))
        with pytest.raises(cg.BackendPanic):
            be.add(x, be.tensor(np.zeros((2, 3), np.uint32)))


@pytest.mark.parametrize("src,dst", [((), (3, 4)), ((4,), (3, 4)), ((3, 1), (3, 4)), ((1, 4), (2, 3, 4)),
                                     ((2, 1, 4), (2, 3, 4)), ((1,), (5,)), ((3, 4), (3, 4))])
def test_broadcast(oracle, dev, src, dst):
    a = rng(7).standard_normal(src).astype(np.float32)
    r, d = both(oracle, dev, lambda be, x: be.broadcast(x, dst), a)
    assert_bits(r[0], d[0])
    assert_bits(r[0], np.broadcast_to(a, dst).astype(np.float32))


def test_broadcast_rejects(cg, oracle, dev):
    for be in (oracle, dev):
        with pytest.raises(cg.ShapeError):
            be.broadcast(be.tensor(np.zeros((3,), np.float32)), (3, 4))
        with pytest.raises(cg.ShapeError):
            be.broadcast(be.tensor(np.zeros((3, 4), np.float32)), (4,))


def test_transpose_reshape_slice_chain(oracle, dev):
    a = rng(8).standard_normal((2, 6, 4, 8)).astype(np.float32)

    def f(be, x):
        t = be.transpose(x, 1, 2)              # [2,4,6,8] view
        s = be.slice(t, 2, 1, 4)               # [2,4,4,8]
        r = be.reshape(s, (8, 32))             # needs a strided pass
        t2 = be.transpose(r, 0, 1)             # [32,8]
        return be.reshape(t2, (4, 8, 8)), be.reshape(x, (12, 32))
    r, d = both(oracle, dev, f, a)
    assert_bits(r[0], d[0])
    assert_bits(r[1], d[1])
    ref = a.transpose(0, 2, 1, 3)[:, :, 1:5, :].reshape(8, 32).T.reshape(4, 8, 8)
    assert_bits(r[0], np.ascontiguousarray(ref))


def test_transpose_materialised_large(oracle, dev):
    a = rng(9).standard_normal((8, 96, 80)).astype(np.float32)
    r, d = both(oracle, dev, lambda be, x: be.reshape(be.transpose(x, 1, 2), (8, 80 * 96)), a)
    assert_bits(r[0], d[0])


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_concat_slice_roundtrip(oracle, dev, dim):
    g = rng(10 + dim)
    sa, sb = [3, 4, 8], [3, 4, 8]
    sb[dim] = 5
    a = g.standard_normal(sa).astype(np.float32)
    b = g.standard_normal(sb).astype(np.float32)
    r, d = both(oracle, dev, lambda be, x, y: be.concat(x, y, dim), a, b)
    assert_bits(r[0], d[0])
    assert_bits(r[0], np.concatenate([a, b], axis=dim))
    r, d = both(oracle, dev,
                lambda be, x, y: be.slice(be.concat(x, y, dim), dim, sa[dim], sb[dim]), a, b)
    assert_bits(d[0], b)


def test_concat_u32_and_views(oracle, dev):
    a = rng(12).integers(0, 1000, (4, 6)).astype(np.uint32)

    def f(be, x):
        return be.concat(be.transpose(x, 0, 1), be.transpose(x, 0, 1), 1)
    r, d = both(oracle, dev, f, a)
    assert_bits(r[0], d[0])
    assert_bits(r[0], np.concatenate([a.T, a.T], axis=1))


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_index_gather(oracle, dev, dim):
    g = rng(20 + dim)
    a = g.standard_normal((9, 7, 12)).astype(np.float32)
    idx = g.integers(0, a.shape[dim], (11,)).astype(np.uint32)
    r, d = both(oracle, dev, lambda be, x, i: be.index(x, dim, i), a, idx)
    assert_bits(r[0], d[0])
    assert_bits(r[0], np.take(a, idx, axis=dim))


def test_index_rank2_indices_are_flattened(oracle, dev):
    g = rng(23)
    a = g.integers(0, 2**32, (10, 4), dtype=np.uint64).astype(np.uint32)
    idx = g.integers(0, 10, (3, 1)).astype(np.uint32)
    r, d = both(oracle, dev, lambda be, x, i: be.index(x, 0, i), a, idx)
    assert r[0].shape == (3, 4)
    assert_bits(r[0], d[0])
    # index(arange(n)) = id
    r, d = both(oracle, dev, lambda be, x: be.index(x, 0, be.arange(10)), a)
    assert_bits(d[0], a)


def test_arange_zeros(cg, oracle, dev):
    for n in (0, 1, 5, 1000):
        r, d = both(oracle, dev, lambda be: be.arange(n))
        assert_bits(r[0], d[0])
        assert_bits(d[0], np.arange(n, dtype=np.uint32))
    for dt, npdt in ((cg.F32, np.float32), (cg.U32, np.uint32)):
        r, d = both(oracle, dev, lambda be: be.zeros((3, 0, 2), dt))
        assert r[0].shape == d[0].shape == (3, 0, 2)
        r, d = both(oracle, dev, lambda be: be.zeros((3, 5), dt))
        assert_bits(d[0], np.zeros((3, 5), npdt))


@pytest.mark.parametrize("shape", [(2, 3), (2, 2, 3), (5, 64), (3, 257), (2, 4096), (1, 9000), (7, 1),
                                   (1, 128256), (3, 40002)])
def test_sum_max_argmax(oracle, dev, shape):
    g = rng(sum(shape))
    a = g.standard_normal(shape).astype(np.float32)
    r, d = both(oracle, dev, lambda be, x: (be.sum(x), be.max(x), be.argmax(x)), a)
    assert r[0].shape == shape[:-1] + (1,)
    absum = np.abs(a).sum(axis=-1, keepdims=True).astype(np.float32)
    assert_close(r[0], d[0], RTOL_F32, scale=absum)
    assert_bits(r[1], d[1])
    assert_bits(r[2], d[2])
    u = g.integers(0, 2**32, shape, dtype=np.uint64).astype(np.uint32)
    r, d = both(oracle, dev, lambda be, x: (be.sum(x), be.max(x), be.argmax(x)), u)
    for i in range(3):
        assert_bits(r[i], d[i])


def test_max_argmax_special_values(oracle, dev):
    nan, inf = np.float32(np.nan), np.float32(np.inf)
    a = np.array([[-inf, -inf, -inf, -inf],       # floor at f32::MIN
                  [nan, 1.0, nan, 0.5],           # NaN ignored by max, +NaN wins argmax
                  [2.0, 7.0, 7.0, 1.0],           # ties -> last index
                  [-0.0, 0.0, -0.0, 0.0],         # +0 > -0 under total_cmp
                  [nan, nan, nan, nan]], dtype=np.float32)
    a[4, 1] = np.frombuffer(np.uint32(0xFFC00000).tobytes(), np.float32)[0]  # -NaN sorts lowest
    r, d = both(oracle, dev, lambda be, x: (be.max(x), be.argmax(x)), a)
    assert_bits(r[0], d[0])
    assert_bits(r[1], d[1])
    assert r[0][0, 0] == np.finfo(np.float32).min
    assert r[0][1, 0] == 1.0 and r[0][4, 0] == np.finfo(np.float32).min
    assert list(r[1].ravel()[:4]) == [3, 2, 2, 3]


@pytest.mark.parametrize("shape,k", [((2, 5), 2), ((4, 60), 4), ((3, 2, 130), 8), ((1, 7), 7), ((5, 9), 1)])
def test_topk(oracle, dev, shape, k):
    g = rng(k)
    a = g.standard_normal(shape).astype(np.float32)
    a.ravel()[::3] = np.float32(0.25)            # many ties
    r, d = both(oracle, dev, lambda be, x: be.topk(x, k), a)
    assert_bits(r[0], d[0])
    assert_bits(r[1], d[1])
    v, i = d
    assert np.all(np.diff(v, axis=-1) <= 0)
    assert_bits(np.take_along_axis(a, i.astype(np.int64), axis=-1), v)


def test_compare(oracle, dev):
    a = rng(30).standard_normal((5, 33)).astype(np.float32)
    b = a.copy()
    b[4, 32] += 1
    n = a.copy()
    n[0, 0] = np.nan
    for be in (oracle, dev):
        ta, tb, tn = be.tensor(a), be.tensor(b), be.tensor(n)
        assert be.compare(ta, be.tensor(a.copy()))
        assert not be.compare(ta, tb)
        assert not be.compare(tn, tn)                    # NaN != NaN
        assert not be.compare(ta, be.reshape(ta, (33, 5)))
        assert be.compare(be.transpose(be.transpose(ta, 0, 1), 0, 1), ta)


MM = [((4, 3), (3, 5)), ((2, 3, 2, 2), (2, 3, 2, 1)), ((1, 130, 70), (1, 70, 200)),
      ((3, 64, 64), (3, 64, 64)), ((1, 1, 96), (1, 96, 300)), ((2, 4, 1, 64), (2, 4, 64, 37)),
      ((1, 5, 257), (1, 257, 9)), ((1, 260, 40), (1, 40, 129))]


@pytest.mark.parametrize("sa,sb", MM)
def test_matmul_f32(oracle, dev, sa, sb):
    g = rng(sum(sa) + sum(sb))
    a = g.standard_normal(sa).astype(np.float32)
    b = g.standard_normal(sb).astype(np.float32)
    r, d = both(oracle, dev, lambda be, x, y: be.matmul(x, y), a, b)
    truth = np.matmul(a.astype(np.float64), b.astype(np.float64))
    scale = np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64))
    assert_close(truth.astype(np.float32), d[0], RTOL_F32, scale=scale)
    assert_close(truth.astype(np.float32), r[0], RTOL_F32, scale=scale)


def test_matmul_reference_vectors(oracle, dev):
    # catgrad/src/interpreter/backend/ndarray.rs:631-674
    a = np.arange(1, 25, dtype=np.float32).reshape(2, 3, 2, 2)
    b = np.arange(1, 13, dtype=np.float32).reshape(2, 3, 2, 1)
    r, d = both(oracle, dev, lambda be, x, y: be.matmul(x, y), a, b)
    exp = np.array([5, 11, 39, 53, 105, 127, 203, 233, 333, 371, 495, 541], np.float32)
    assert_bits(r[0].ravel(), exp)
    assert_bits(d[0].ravel(), exp)


@pytest.mark.parametrize("m,k,n", [(1, 64, 48), (1, 2048, 512), (4, 256, 100), (8, 96, 64), (130, 72, 36),
                                   (1, 300, 77)])
def test_matmul_transposed_operands(oracle, dev, m, k, n):
    """The `linear` pattern: W[out,in] -> transpose -> reshape [1,in,out] -> matmul, and K^T."""
    g = rng(m * k + n)
    x = g.standard_normal((1, m, k)).astype(np.float32)
    w = g.standard_normal((n, k)).astype(np.float32)

    def f(be, x, w):
        wt = be.reshape(be.transpose(w, 0, 1), (1, k, n))
        y = be.matmul(x, wt)
        # lhs transposed as well: (y^T)^T through a view
        xt = be.transpose(be.reshape(be.transpose(x, 1, 2), (1, k, m)), 1, 2)
        return y, be.matmul(xt, wt)
    r, d = both(oracle, dev, f, x, w)
    truth = np.matmul(x.astype(np.float64), w.T.astype(np.float64))
    scale = np.matmul(np.abs(x).astype(np.float64), np.abs(w.T).astype(np.float64))
    assert_close(truth.astype(np.float32), d[0], RTOL_F32, scale=scale)
    assert_close(truth.astype(np.float32), d[1], RTOL_F32, scale=scale)


def test_matmul_u32_and_errors(cg, oracle, dev):
    g = rng(40)
    a = g.integers(0, 2**32, (2, 5, 7), dtype=np.uint64).astype(np.uint32)
    b = g.integers(0, 2**32, (2, 7, 3), dtype=np.uint64).astype(np.uint32)
    r, d = both(oracle, dev, lambda be, x, y: be.matmul(x, y), a, b)
    assert_bits(r[0], d[0])
    for be in (oracle, dev):
        with pytest.raises(cg.ShapeError, match="incompatible matrix dimensions"):
            be.matmul(be.tensor(np.zeros((2, 3), np.float32)), be.tensor(np.zeros((4, 2), np.float32)))
        with pytest.raises(cg.ShapeError, match="batch dimensions must match"):
            be.matmul(be.tensor(np.zeros((2, 2, 3), np.float32)), be.tensor(np.zeros((3, 3, 2), np.float32)))
        with pytest.raises(cg.ShapeError):
            be.matmul(be.tensor(np.zeros((3,), np.float32)), be.tensor(np.zeros((3, 2), np.float32)))


def test_fused_chain_matches_op_by_op(oracle, hip, hip_eager):
    """A long elementwise tree with broadcasts: deferred+fused == eager == oracle."""
    g = rng(50)
    x = g.standard_normal((3, 17, 32)).astype(np.float32)
    w = g.standard_normal((32,)).astype(np.float32)

    def f(be, x, w):
        one = be.broadcast(be.ndarray_from_vec_f32([1.0], ()), x.shape)
        e = be.broadcast(be.ndarray_from_vec_f32([2.7182817], ()), x.shape)
        half = be.broadcast(be.ndarray_from_vec_f32([0.5], ()), x.shape)
        sig = be.div(one, be.add(one, be.pow(e, be.neg(x))))       # sigmoid
        y = be.mul(be.mul(x, sig), be.broadcast(w, x.shape))        # silu * w
        s = be.sum(be.mul(y, y))                                    # reduce with prologue
        z = be.div(y, be.broadcast(be.pow(be.add(s, be.slice(be.sum(half), 2, 0, 1)),
                                          be.slice(half, 2, 0, 1)), x.shape))
        return z, s
    r, d = both(oracle, hip, f, x, w)
    _, e = both(oracle, hip_eager, f, x, w)
    assert_close(r[0], d[0], RTOL_F32)
    assert_close(r[0], e[0], RTOL_F32)
    assert_close(r[1], d[1], RTOL_F32)


def test_bf16_mode_matmul(cg, oracle, hip_bf16):
    g = rng(60)
    for (m, k, n) in [(1, 512, 256), (96, 256, 200), (4, 128, 64)]:
        x = g.standard_normal((1, m, k)).astype(np.float32)
        w = (g.standard_normal((n, k)) * 0.05).astype(np.float32)

        def f(be, x, w):
            return be.matmul(x, be.reshape(be.transpose(w, 0, 1), (1, k, n)))
        r, d = both(oracle, hip_bf16, f, x, w)
        scale = np.matmul(np.abs(x), np.abs(w.T))
        assert_close(r[0], d[0], RTOL_BF16, scale=scale)
    # rank-2 parameters are stored as bf16: reading them back gives RNE-rounded values
    w = g.standard_normal((8, 16)).astype(np.float32)
    back = hip_bf16.numpy(hip_bf16.tensor(w))
    u = w.view(np.uint32).astype(np.uint64)
    rne = (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)
    assert_bits(back, rne)
    # gather from a bf16 table widens exactly
    idx = np.array([3, 0, 7, 3], np.uint32)
    got = hip_bf16.numpy(hip_bf16.index(hip_bf16.tensor(w), 0, hip_bf16.tensor(idx)))
    assert_bits(got, rne[idx])


@pytest.mark.gpu
def test_bf16_mode_matmul_shape_sweep(oracle, hip_bf16):
    """Many-row products in bf16 mode across the shapes that select different GEMM variants (tile
    sizes, two or four LDS stages, split-K, tails in every dimension, batches), against the oracle on
    operands already rounded to bf16."""
    import vectors
    g = rng(61)
    shapes = [(1, 64, 64, 64), (1, 64, 128, 128), (1, 100, 192, 200), (1, 512, 320, 512), (1, 130, 1024, 192),
              (1, 256, 2048, 256), (1, 1024, 64, 1024), (1, 2048, 256, 2048), (3, 200, 128, 136), (2, 64, 4096, 64),
              (1, 72, 72, 72), (1, 512, 8192, 128)]       # batch, M, K, N
    for (b, m, k, n) in shapes:
        x = vectors.bf16_round(g.standard_normal((b, m, k)).astype(np.float32))
        w = vectors.bf16_round((g.standard_normal((b, n, k)) * 0.05).astype(np.float32))

        def f(be, x, w):
            x = be.add(x, be.sub(x, x))                      # a computed f32 value
            return be.matmul(x, be.transpose(w, 1, 2))
        r, d = both(oracle, hip_bf16, f, x, w)
        scale = np.matmul(np.abs(x), np.abs(np.swapaxes(w, 1, 2)))
        assert_close(r[0], d[0], RTOL_BF16, scale=scale)


@pytest.mark.gpu
def test_small_f32_matmul_layouts_and_tails(oracle, hip):
    """Products of a few 32 x 32 tiles in f32 (the layers of a small MLP): either operand with unit
    stride along k or along its other axis, sizes that leave tails in M, N and K (K below and across
    the 32-wide chunks, not a multiple of 4, deep enough to be split over workgroups), batches, a broadcast right
    operand and a sliced left one."""
    g = rng(62)
    shapes = [(1, 9, 1, 1), (1, 33, 5, 31), (1, 64, 256, 10), (1, 64, 128, 256), (1, 70, 300, 70), (1, 17, 37, 130),
              (3, 40, 129, 50), (2, 100, 1000, 12), (1, 32, 4096, 32), (1, 12, 3, 300), (1, 11, 2048, 9),
              (2, 64, 8200, 64)]       # batch, M, K, N; the deep ones are split along k
    for (b, m, k, n) in shapes:
        x = g.standard_normal((b, m, k)).astype(np.float32)
        w = g.standard_normal((b, k, n)).astype(np.float32)
        xt = np.ascontiguousarray(np.swapaxes(x, 1, 2))
        wt = np.ascontiguousarray(np.swapaxes(w, 1, 2))
        xpad = g.standard_normal((b, m, k + 3)).astype(np.float32)

        def f(be, x, w, xt, wt, xpad):
            y0 = be.matmul(x, w)                                             # A along k, B along n
            y1 = be.matmul(x, be.transpose(wt, 1, 2))                        # both along k
            y2 = be.matmul(be.transpose(xt, 1, 2), w)                        # neither
            y3 = be.matmul(be.transpose(xt, 1, 2), be.transpose(wt, 1, 2))   # A along m, B along k
            y4 = be.matmul(be.slice(xpad, 2, 1, k), w)                       # rows that start off 16-byte alignment
            w0 = be.broadcast(be.slice(w, 0, 0, 1), (b, k, n))               # one matrix for every batch
            return y0, y1, y2, y3, y4, be.matmul(x, w0)
        r, d = both(oracle, hip, f, x, w, xt, wt, xpad)
        truth = np.matmul(x.astype(np.float64), w.astype(np.float64))
        scale = np.matmul(np.abs(x).astype(np.float64), np.abs(w).astype(np.float64))
        for i in range(4):
            assert_close(truth.astype(np.float32), d[i], RTOL_F32, scale=scale)
        xs = xpad[:, :, 1:1 + k].astype(np.float64)
        assert_close(np.matmul(xs, w.astype(np.float64)).astype(np.float32), d[4], RTOL_F32,
                     scale=np.matmul(np.abs(xs), np.abs(w).astype(np.float64)))
        w0 = np.broadcast_to(w[:1], w.shape).astype(np.float64)
        assert_close(np.matmul(x.astype(np.float64), w0).astype(np.float32), d[5], RTOL_F32,
                     scale=np.matmul(np.abs(x).astype(np.float64), np.abs(w0)))
        for i in range(6):
            assert_close(r[i], d[i], 2 * RTOL_F32, scale=scale if i != 4 else np.matmul(np.abs(xs), np.abs(w).astype(np.float64)))


def test_row_fusion_layernorm_and_softmax_views(oracle, hip, hip_eager):
    """Row programs (reduction stages + final segment in one kernel) on strided inputs: softmax of
    a transposed view, layernorm with gamma/beta broadcasts, and a row value read twice."""
    import vectors
    lang, nn, helpers = vectors.lang, vectors.nn, vectors.helpers
    g = rng(70)
    x = (g.standard_normal((2, 24, 40)) * 3).astype(np.float32)
    gamma = g.standard_normal((40,)).astype(np.float32)

    def f(b, x, gamma):
        xt = lang.transpose(b, 1, 2, x)                         # [2, 40, 24] view
        sm = nn.softmax(b, xt)
        ln = helpers.layernorm_raw(b, 1e-5, x)
        ln = ln * lang.broadcast(b, gamma, lang.shape(b, ln))
        m = lang.max(b, x)
        twice = (x - lang.broadcast(b, m, lang.shape(b, x))) * lang.broadcast(b, m, lang.shape(b, x))
        return sm, ln, twice
    ref = vectors.run(oracle, f, 3, x, gamma)
    for dev in (hip, hip_eager):
        got = vectors.run(dev, f, 3, x, gamma)
        for r, d in zip(ref, got):
            assert np.allclose(d, r, rtol=1e-4, atol=2e-6)


def test_concat_append_in_place_keeps_values(dev):
    """The KV-cache pattern: repeated concat of one row onto a growing tensor.  Storage may be
    reused in place only when nobody else holds the old value."""
    g = rng(80)
    cur = g.standard_normal((1, 2, 8, 4)).astype(np.float32)
    t = dev.tensor(cur)
    held = []
    for step in range(40):
        y = g.standard_normal((1, 2, 1, 4)).astype(np.float32)
        new = dev.concat(t, dev.tensor(y), 2)
        cur = np.concatenate([cur, y], axis=2)
        if step % 3 == 0:
            held.append((t, cur[:, :, :-1].copy()))     # an old value somebody still reads
        t = new
        if step % 5 == 0:
            assert_bits(dev.numpy(t), cur)
    assert_bits(dev.numpy(t), cur)
    for old, exp in held:
        assert_bits(dev.numpy(old), exp)
    # the grown tensor is an ordinary value: views and matmuls read it through its strides
    w = g.standard_normal((1, 2, 4, 3)).astype(np.float32)
    out = dev.numpy(dev.matmul(t, dev.tensor(w)))
    assert np.allclose(out, np.matmul(cur, w), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("view", ["transposed", "regrouped", "sliced"])
def test_concat_onto_another_view_of_a_cache_copies(oracle, dev, view):
    """A sole-owner view of a cache's storage that does not walk it like the cache (a transpose, a
    reshape that merges rows and columns) must not be appended to in place: its "next row" lies on
    live elements, or past the room of a head."""
    g = rng(("view", view))
    base = g.standard_normal((1, 2, 8, 4)).astype(np.float32)
    first = g.standard_normal((1, 2, 1, 4)).astype(np.float32)
    cache_np = np.concatenate([base, first], axis=2)                   # [1, 2, 9, 4], storage with spare rows
    outs = []
    for be in (oracle, dev):
        t = be.concat(be.tensor(base), be.tensor(first), 2)
        be.to_vec(t)                                                   # in memory now
        if view == "transposed":
            v, v_np = be.transpose(t, 2, 3), cache_np.transpose(0, 1, 3, 2)            # [1, 2, 4, 9]
        elif view == "regrouped":
            v, v_np = be.reshape(t, (1, 2, 3, 12)), cache_np.reshape(1, 2, 3, 12)
        else:
            v, v_np = be.slice(t, 3, 0, 2), cache_np[..., :2]                          # walks it like the cache
        be.to_vec(v)
        del t                                                          # the view is the only owner left
        y = g.standard_normal(v_np.shape[:2] + (1,) + v_np.shape[3:]).astype(np.float32) if be is oracle else y
        r = be.concat(v, be.tensor(y), 2)
        del v
        outs.append(be.numpy(r))
        assert_bits(outs[-1], np.concatenate([v_np, y], axis=2))
    assert_bits(outs[0], outs[1])


def test_repeat_kv_matmul(oracle, dev):
    """q @ repeat_kv(k)^T and p @ repeat_kv(v) (helpers.rs:147-161, models/llama.rs:95-108)."""
    import vectors
    lang, helpers = vectors.lang, vectors.helpers
    g = rng(81)
    for s, t in ((1, 37), (5, 5), (70, 70)):
        q = g.standard_normal((1, 8, s, 16)).astype(np.float32)
        k = g.standard_normal((1, 2, t, 16)).astype(np.float32)
        p = g.standard_normal((1, 8, s, t)).astype(np.float32)

        def f(b, q, k, p):
            kr = helpers.repeat_kv(b, 4, k)
            return lang.matmul(b, q, lang.transpose(b, 2, 3, kr)), lang.matmul(b, p, kr)
        ref = vectors.run(oracle, f, 2, q, k, p)
        got = vectors.run(dev, f, 2, q, k, p)
        kr = np.repeat(k, 4, axis=1)
        assert np.allclose(ref[0], q @ kr.transpose(0, 1, 3, 2), rtol=1e-4, atol=1e-4)
        for r, d in zip(ref, got):
            assert np.allclose(d, r, rtol=1e-4, atol=1e-4)


def test_one_row_matmuls_sharing_x_go_out_together(oracle, hip, hip_bf16):
    """q/k/v- and gate/up-style linears on one activation row: one launch, same results."""
    g = rng(82)
    k = 1024
    x = g.standard_normal((1, 1, k)).astype(np.float32)
    ws = [(g.standard_normal((n, k)) * 0.05).astype(np.float32) for n in (96, 40, 1024)]

    def f(be, x, *w):
        x = be.reshape(x, (1, 1, k))      # uploaded as rank 1: an activation, kept f32 in bf16 mode
        outs = [be.matmul(x, be.reshape(be.transpose(wi, 0, 1), (1, k, wi.shape[0]))) for wi in w]
        return tuple(outs)
    for dev, tol in ((hip, RTOL_F32), (hip_bf16, RTOL_BF16)):
        dev.trace(True)
        dev.trace_reset()
        r, d = both(oracle, dev, f, x.reshape(k), *ws)
        rep = dev.trace_report()
        dev.trace(False)
        name = "gemv_rowdot_f32" if dev is hip else "gemv_rowdot_bf16"
        assert rep[name]["launches"] == 1, rep
        for ref, got, w in zip(r, d, ws):
            assert_close(ref, got, tol, scale=np.abs(x) @ np.abs(w.T) + 1e-6)

"""The hand-written pattern kernels (softmax, RMSNorm, RoPE, SwiGLU/GeGLU, single binary op):
each is checked against the oracle, against the generic program path on the same device, and
for having actually been dispatched (by kernel name in the backend's trace)."""
import numpy as np
import pytest

import vectors

pytestmark = pytest.mark.gpu
lang, nn, helpers = vectors.lang, vectors.nn, vectors.helpers


def run_traced(be, fn, n_out, *arrays, params=None):
    be.trace(True)
    be.trace_reset()
    out = vectors.run(be, fn, n_out, *arrays, params=params)
    rep = be.trace_report()
    be.trace(False)
    return out, set(rep)


def check(oracle, hip, hip_nopat, fn, n_out, arrays, kernel, params=None, rtol=1e-4, atol=1e-6):
    ref = vectors.run(oracle, fn, n_out, *arrays, params=params)
    got, names = run_traced(hip, fn, n_out, *arrays, params=params)
    gen, gnames = run_traced(hip_nopat, fn, n_out, *arrays, params=params)
    assert kernel in names, f"{kernel} not dispatched: {sorted(names)}"
    assert kernel not in gnames
    for r, g, h in zip(ref, got, gen):
        assert np.allclose(g, r, rtol=rtol, atol=atol), np.abs(g - r).max()
        assert np.allclose(h, r, rtol=rtol, atol=atol), np.abs(h - r).max()


@pytest.mark.parametrize("shape", [(1, 1, 2048), (1, 7, 64), (2, 33, 1152), (1, 3, 8192), (5, 16),
                                   # thousands of rows: a wave per row, several rows per workgroup
                                   (1, 2050, 1152), (2, 1025, 256), (1, 2049, 2048), (1, 2051, 512), (1, 2048, 1024),
                                   (1, 2053, 64), (1, 2049, 2052)])
def test_rmsnorm(oracle, hip, hip_nopat, shape):
    g = np.random.default_rng(sum(shape))
    x = (g.standard_normal(shape) * 3).astype(np.float32)
    if len(shape) == 2:
        x = x.reshape((1,) + shape)
    gamma = g.standard_normal(shape[-1]).astype(np.float32)
    p = {"n.weight": gamma}
    check(oracle, hip, hip_nopat, lambda b, v: helpers.rmsnorm(b, 1e-5, lang.path(["n"]), v), 1, [x],
          "rmsnorm_fused", params=p)
    check(oracle, hip, hip_nopat, lambda b, v: helpers.rmsnorm_raw(b, 1e-6, v), 1, [x], "rmsnorm_fused")

    def gemma(b, v):  # lr * (one + gamma), catgrad-llm/src/models/gemma3.rs:60-68
        gm = lang.param(b, lang.path(["n", "weight"]))
        lr = helpers.rmsnorm_raw(b, 1e-6, v)
        gm = lang.broadcast(b, gm, lang.shape(b, lr))
        one = lang.constant(b, 1.0, lang.shape(b, gm))
        return lr * (one + gm)
    check(oracle, hip, hip_nopat, gemma, 1, [x], "rmsnorm_fused", params=p)


def test_rmsnorm_of_strided_rows(oracle, hip, hip_nopat):
    g = np.random.default_rng(3)
    x = g.standard_normal((1, 6, 40, 32)).astype(np.float32)

    def f(b, v):  # QK-norm style: rows are slices of a wider tensor
        s = lang.slice(b, 3, 0, 16, v)
        s = lang.reshape(b, lang.make_shape(b, 1, 240, 16), s)
        return helpers.rmsnorm_raw(b, 1e-6, s)
    check(oracle, hip, hip_nopat, f, 1, [x], "rmsnorm_fused")


@pytest.mark.parametrize("dims", [(2, 40, 4, 64), (3, 5, 2, 256), (1, 7, 3, 32), (2, 9, 1, 64), (2, 301, 4, 64)])
def test_rmsnorm_of_rows_behind_a_head_transpose(oracle, hip, hip_nopat, dims):
    """gemma3.rs:99-117 norms q and k after the head transpose, folded to [b * heads * s, head_dim] - a
    reshape that strides cannot express.  The kernel reads the rows where the projection left them;
    nothing is copied into row-major order first."""
    B, S, H, D = dims
    g = np.random.default_rng(B * S + H)
    x = (g.standard_normal((B, S, H * D)) * 2).astype(np.float32)
    p = {"n.weight": (g.standard_normal(D) * 0.3).astype(np.float32)}

    def f(b, v):
        v = v + v - v
        q = lang.transpose(b, 1, 2, lang.reshape(b, lang.make_shape(b, B, S, H, D), v))
        q = lang.reshape(b, lang.make_shape(b, B * H * S, D), q)
        gm = lang.param(b, lang.path(["n", "weight"]))
        lr = helpers.rmsnorm_raw(b, 1e-6, lang.reshape(b, lang.make_shape(b, 1, B * H * S, D), q))
        gm = lang.broadcast(b, gm, lang.shape(b, lr))
        q = lr * (lang.constant(b, 1.0, lang.shape(b, gm)) + gm)
        return lang.reshape(b, lang.make_shape(b, B, H, S, D), q)
    check(oracle, hip, hip_nopat, f, 1, [x], "rmsnorm_fused", params=p, rtol=1e-4, atol=1e-5)
    _, names = run_traced(hip, f, 1, x, params=p)
    assert "ew_copy" not in names, sorted(names)
    (ref,) = vectors.run(oracle, f, 1, x, params=p)
    xr = x.reshape(B, S, H, D).transpose(0, 2, 1, 3).astype(np.float64)
    want = xr / np.sqrt((xr * xr).mean(-1, keepdims=True) + 1e-6) * (1 + p["n.weight"].astype(np.float64))
    assert np.allclose(ref, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("extra_reader", [False, True])
def test_rmsnorm_written_for_the_gemms_that_wait_for_it(oracle, hip_bf16, extra_reader):
    """bf16 mode, many rows: a norm whose only readers are products is written as bf16 alone (the form
    the GEMMs read); with any other reader it is written as f32 with a bf16 copy beside it."""
    M, K, N = 192, 256, 128
    g = np.random.default_rng(M + extra_reader)
    x = vectors.bf16_round((g.standard_normal((1, M, K)) * 2).astype(np.float32))  # (matrices are uploaded as bf16)
    p = {"n.weight": g.standard_normal(K).astype(np.float32)}
    for nm in ("q", "k"):
        p[nm + ".weight"] = vectors.bf16_round((g.standard_normal((N, K)) * 0.05).astype(np.float32))

    def f(b, v):
        v = v + v - v
        h = helpers.rmsnorm(b, 1e-5, lang.path(["n"]), v)
        q, k = (nn.linear_no_bias(b, K, N, lang.path([nm]), h) for nm in ("q", "k"))
        return (q, k, h * h) if extra_reader else (q, k)
    n_out = 3 if extra_reader else 2
    ref = vectors.run(oracle, f, n_out, x, params=p)
    hip_bf16.trace(2)
    hip_bf16.trace_reset()
    got = vectors.run(hip_bf16, f, n_out, x, params=p)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    norms = [k for k in rep if k.startswith("rmsnorm_fused")]
    assert norms == [f"rmsnorm_fused[{M}x{K},{'f32+bf16' if extra_reader else 'bf16'}]"], sorted(rep)
    assert not any(k.startswith("cast") or "narrow" in k for k in rep), sorted(rep)
    for r, d in zip(ref[:2], got[:2]):
        assert d.shape == r.shape and np.max(np.abs(d - r)) <= 2e-2 * np.abs(r).max()
    if extra_reader:  # the other reader sees the f32 values
        assert np.allclose(got[2], ref[2], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", [(1, 32, 1, 530), (1, 4, 19, 19), (2, 3, 64, 512), (1, 2, 5, 1500),
                                   (1, 1, 3, 5000), (3, 60)])
def test_softmax(oracle, hip, hip_nopat, shape):
    g = np.random.default_rng(sum(shape))
    x = (g.standard_normal(shape) * 4).astype(np.float32)
    check(oracle, hip, hip_nopat, nn.softmax, 1, [x], "softmax_fused", atol=1e-7)

    def scaled(b, a):
        return nn.softmax(b, a / lang.constant(b, 8.0, lang.shape(b, a)))
    check(oracle, hip, hip_nopat, scaled, 1, [x], "softmax_fused", atol=1e-7)


@pytest.mark.parametrize("s,t", [(19, 19), (64, 64), (1, 530)])
def test_softmax_scale_and_causal_mask(oracle, hip, hip_nopat, s, t):
    """attention's `attn / sqrt(d) + broadcast(causal_mask)` (models/llama.rs:97-107); with s = 1
    the mask folds to the constant -0.0."""
    g = np.random.default_rng(s * t)
    x = (g.standard_normal((1, 6, s, t)) * 5).astype(np.float32)

    def f(b, a):
        sh = lang.shape(b, a)
        _, _, n, _ = lang.unpack(b, 4, sh)
        a = a / lang.constant(b, 8.0, sh)
        mask = lang.broadcast(b, helpers.causal_mask(b, n), sh)
        return nn.softmax(b, a + mask)
    check(oracle, hip, hip_nopat, f, 1, [x], "softmax_fused", atol=1e-7)


@pytest.mark.parametrize("b,h,s,d,pos", [(1, 32, 1, 64, 17), (1, 8, 24, 64, 0), (2, 4, 9, 256, 3)])
def test_rope(oracle, hip, hip_nopat, b, h, s, d, pos):
    g = np.random.default_rng(b + h + s + d)
    x = g.standard_normal((b, s, h, d)).astype(np.float32)     # as the q projection leaves it

    def f(bl, v):
        cos, sin = helpers.rope_tables(bl, 500000.0, lang.to_nat(bl, pos + s + 5), d)
        q = lang.transpose(bl, 1, 2, v)                         # [b, h, s, d] view
        return helpers.apply_rope_embedding(bl, pos, d, cos, sin, q)
    check(oracle, hip, hip_nopat, f, 1, [x], "rope_fused", atol=2e-6)


@pytest.mark.parametrize("shape", [(1, 1, 8192), (1, 37, 256), (2, 5, 6912)])
def test_swiglu_geglu(oracle, hip, hip_nopat, shape):
    g = np.random.default_rng(shape[-1])
    gate = (g.standard_normal(shape) * 3).astype(np.float32)
    up = g.standard_normal(shape).astype(np.float32)
    check(oracle, hip, hip_nopat, lambda b, x, y: nn.silu(b, x) * y, 1, [gate, up], "swiglu_fused")
    check(oracle, hip, hip_nopat, lambda b, x, y: nn.gelu(b, x) * y, 1, [gate, up], "geglu_fused",
          atol=2e-6)


def test_single_binary_op(oracle, hip, hip_nopat):
    g = np.random.default_rng(9)
    x = g.standard_normal((4, 96, 128)).astype(np.float32)
    y = g.standard_normal((4, 96, 128)).astype(np.float32)
    bias = g.standard_normal((128,)).astype(np.float32)
    check(oracle, hip, hip_nopat, lambda b, p, q: p + q, 1, [x, y], "binary_f32", rtol=0, atol=0)
    check(oracle, hip, hip_nopat, lambda b, p, q: p / q, 1, [x, y], "binary_f32", rtol=0, atol=0)
    check(oracle, hip, hip_nopat, lambda b, p, v: p + lang.broadcast(b, v, lang.shape(b, p)), 1, [x, bias],
          "binary_f32", rtol=0, atol=0)


def test_near_misses_take_the_generic_path(oracle, hip):
    """A softmax whose max is read elsewhere, an rmsnorm with a different exponent: same results
    through the generic programs."""
    g = np.random.default_rng(10)
    x = (g.standard_normal((2, 9, 40)) * 2).astype(np.float32)

    def f(b, v):
        sh = lang.shape(b, v)
        m = lang.max(b, v)
        e = nn.exp(b, v - lang.broadcast(b, m, sh))
        s = lang.sum(b, e)
        return e / lang.broadcast(b, s, sh), m          # m escapes
    ref = vectors.run(oracle, f, 2, x)
    got, names = run_traced(hip, f, 2, x)
    assert "softmax_fused" not in names
    for r, d in zip(ref, got):
        assert np.allclose(d, r, rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("shape", [(1, 2048, 2048), (1, 8192, 2048), (1, 72, 40), (3, 512, 64)])  # M, K, N
@pytest.mark.parametrize("order", ["res_first", "mm_first"])
def test_residual_add_in_gemv_epilogue(oracle, hip, hip_nopat, shape, order):
    """res + linear(x) on one-row activations: no separate add launch, same values."""
    M, K, N = shape
    g = np.random.default_rng(K + N)
    x = g.standard_normal((1, M, K)).astype(np.float32)
    w = (g.standard_normal((N, K)) * 0.05).astype(np.float32)
    res = g.standard_normal((1, M, N)).astype(np.float32)

    def f(b, xv, rv):
        xv = xv + xv - xv
        y = nn.linear_no_bias(b, K, N, lang.path(["l"]), xv)
        return rv + y if order == "res_first" else y + rv
    p = {"l.weight": w}
    (ref,) = vectors.run(oracle, f, 1, x, res, params=p)
    got, names = run_traced(hip, f, 1, x, res, params=p)
    (gen,) = vectors.run(hip_nopat, f, 1, x, res, params=p)
    if M == 1:
        assert "binary_f32" not in names, sorted(names)
    assert np.allclose(got[0], ref, rtol=1e-4, atol=1e-5)
    assert np.allclose(gen, ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", [(512, 2048, (2048, 512, 512)), (130, 256, (256, 128, 384)), (64, 64, (128, 128, 128))])
def test_sibling_products_as_one_grouped_gemm(oracle, hip_bf16, shape):
    """bf16 mode, many rows: q_proj, k_proj, v_proj of one input go out as one launch; each product
    lands in its own tensor."""
    M, K, Ns = shape
    g = np.random.default_rng(M + K)
    x = vectors.bf16_round(g.standard_normal((1, M, K)).astype(np.float32))
    p = {f"w{i}.weight": vectors.bf16_round((g.standard_normal((n, K)) * 0.05).astype(np.float32)) for i, n in enumerate(Ns)}

    def f(b, xv):
        xv = xv + xv - xv
        return tuple(nn.linear_no_bias(b, K, n, lang.path([f"w{i}"]), xv) for i, n in enumerate(Ns))
    ref = vectors.run(oracle, f, 3, x, params=p)
    hip_bf16.trace(2)
    hip_bf16.trace_reset()
    got = vectors.run(hip_bf16, f, 3, x, params=p)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    gemms = {k: v["launches"] for k, v in rep.items() if k.startswith("gemm_mfma_bf16")}
    assert sum(gemms.values()) == 1 and "grouped" in next(iter(gemms)), gemms
    for r, d in zip(ref, got):
        assert d.shape == r.shape and np.max(np.abs(d - r)) <= 2e-2 * np.abs(r).max()


def test_sibling_products_of_a_batch_folded_per_linear(oracle, hip_bf16):
    """bf16 mode, a batch of prompts: every linear folds the batch into the rows with a reshape of its
    own, so q_proj, k_proj, v_proj read three nodes that are one matrix in memory; they still go out
    as one launch."""
    B, S, K, Ns = 4, 96, 256, (256, 128, 128)
    g = np.random.default_rng(B * S)
    x = vectors.bf16_round(g.standard_normal((B, S, K)).astype(np.float32))
    p = {f"w{i}.weight": vectors.bf16_round((g.standard_normal((n, K)) * 0.05).astype(np.float32)) for i, n in enumerate(Ns)}

    def f(b, xv):
        xv = xv + xv - xv
        return tuple(_folded_linear(b, K, n, f"w{i}", xv) for i, n in enumerate(Ns))
    ref = vectors.run(oracle, f, 3, x, params=p)
    hip_bf16.trace(2)
    hip_bf16.trace_reset()
    got = vectors.run(hip_bf16, f, 3, x, params=p)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    gemms = {k: v["launches"] for k, v in rep.items() if k.startswith("gemm_mfma_bf16")}
    assert sum(gemms.values()) == 1 and "grouped" in next(iter(gemms)), gemms
    for r, d in zip(ref, got):
        assert d.shape == r.shape and np.max(np.abs(d - r)) <= 2e-2 * np.abs(r).max()


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("shape", [(256, 512, 1024), (200, 256, 384), (100, 192, 160), (2100, 128, 3080)])  # rows, K, N
def test_gated_activation_in_the_gemm_epilogue(oracle, hip_bf16, shape, act):
    """bf16 mode, many rows: act(gate_proj(x)) * up_proj(x) as one GEMM over both weight matrices with the
    activation applied where the two products sit in registers (neither is stored), followed by down_proj
    reading the bf16 copy that GEMM wrote."""
    *rows, K, N = shape
    g = np.random.default_rng(K + N)
    x = vectors.bf16_round(g.standard_normal((*rows, K) if len(rows) > 1 else (1, *rows, K)).astype(np.float32))
    p = {"g.weight": vectors.bf16_round((g.standard_normal((N, K)) * 0.05).astype(np.float32)),
         "u.weight": vectors.bf16_round((g.standard_normal((N, K)) * 0.05).astype(np.float32)),
         "d.weight": vectors.bf16_round((g.standard_normal((K, N)) * 0.05).astype(np.float32))}

    def f(b, xv):
        xv = xv + xv - xv
        gt = nn.linear_no_bias(b, K, N, lang.path(["g"]), xv)
        up = nn.linear_no_bias(b, K, N, lang.path(["u"]), xv)
        h = (nn.silu(b, gt) if act == "silu" else nn.gelu(b, gt)) * up
        return nn.linear_no_bias(b, N, K, lang.path(["d"]), h), h
    ref = vectors.run(oracle, f, 2, x, params=p)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    got = vectors.run(hip_bf16, f, 2, x, params=p)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    launches = {k: v["launches"] for k, v in rep.items()}
    # x + x - x, two GEMMs, nothing else: no activation kernel, no generic program, no narrowing pass for h
    assert launches.get("gemm_mfma_bf16") == 2 and launches.get("ew_fused") == 1, launches
    # (ew_to_bf16: the uploads of x and the three weights; ew_copy: h is stored as bf16 only and this test reads it back)
    assert set(launches) <= {"gemm_mfma_bf16", "ew_fused", "cast_bf16", "ew_to_bf16", "ew_copy"}, launches
    assert launches.get("cast_bf16", 0) <= 1 and launches.get("ew_copy", 0) <= 1, launches
    for r, d in zip(ref, got):
        assert np.max(np.abs(d - r)) <= 2e-2 * np.abs(r).max()


@pytest.mark.parametrize("shape", [(256, 2048, 512), (512, 8192, 2048), (130, 1024, 192), (2048, 2048, 2048)])  # M, K, N
def test_residual_add_with_a_split_gemm(oracle, hip_bf16, shape):
    """bf16 mode, many rows: when the product is split along k, the pass that sums the slices adds the
    residual; otherwise the generic add runs.  Same values either way."""
    M, K, N = shape
    g = np.random.default_rng(M + K + N)
    x = vectors.bf16_round(g.standard_normal((1, M, K)).astype(np.float32))
    w = vectors.bf16_round((g.standard_normal((N, K)) * 0.05).astype(np.float32))
    res = g.standard_normal((1, M, N)).astype(np.float32)

    def f(b, xv, rv):
        xv = xv + xv - xv
        y = nn.linear_no_bias(b, K, N, lang.path(["l"]), xv)
        rv = lang.reshape(b, lang.shape(b, y), rv)      # the residual stream: an f32 value in memory
        return rv + y
    p = {"l.weight": w}
    res = res.reshape(-1)                               # rank 1: stays f32 in bf16 mode
    (ref,) = vectors.run(oracle, f, 1, x, res, params=p)
    got, names = run_traced(hip_bf16, f, 1, x, res, params=p)
    assert "gemm_mfma_bf16" in names
    if shape in ((256, 2048, 512), (512, 8192, 2048)):        # few tiles, deep k: split
        assert "binary_f32" not in names, sorted(names)
    assert np.max(np.abs(got[0] - ref)) <= 2e-2 * np.abs(ref).max()


@pytest.mark.parametrize("shape", [(512, 8192, 2048), (256, 2048, 512), (512, 2048, 2048), (100, 4096, 264)])  # M, K, N
@pytest.mark.parametrize("mode", ["bf16", "f32"])
def test_norm_that_sums_the_slices_of_a_split_gemm(hip, hip_bf16, shape, mode):
    """`residual + linear(x)` over many rows closes a decoder block (models/llama.rs:166-186) and an RMSNorm
    reads it next.  When the product is split along k, the block end stays the slices of the product and the
    norm sums them (and the residual) on its way in, storing the sum for its other readers: the bits of the
    same two blocks run as two programs, where the sum is a pass of its own."""
    be = hip_bf16 if mode == "bf16" else hip
    M, K, N = shape
    g = np.random.default_rng(M + K + N)
    x = vectors.bf16_round(g.standard_normal((1, M, K)).astype(np.float32))
    p = {"a.weight": vectors.bf16_round((g.standard_normal((N, K)) * 0.05).astype(np.float32)),
         "b.weight": vectors.bf16_round((g.standard_normal((N, N)) * 0.05).astype(np.float32)),
         "n.weight": g.standard_normal(N).astype(np.float32)}
    res = g.standard_normal(M * N).astype(np.float32)   # rank 1: stays f32 in bf16 mode

    def first(b, xv, rv):
        xv = xv + xv - xv
        y = nn.linear_no_bias(b, K, N, lang.path(["a"]), xv)
        return lang.reshape(b, lang.shape(b, y), rv) + y

    def second(b, hv):
        return hv + nn.linear_no_bias(b, N, N, lang.path(["b"]), helpers.rmsnorm(b, 1e-5, lang.path(["n"]), hv))

    def second_alone(b, hv):
        return second(b, lang.reshape(b, lang.make_shape(b, 1, M, N), hv))

    def both(b, xv, rv):
        h = first(b, xv, rv)
        return second(b, h), h
    (h_alone,) = vectors.run(be, first, 1, x, res, params=p)
    (h2_alone,) = vectors.run(be, second_alone, 1, h_alone.reshape(-1), params=p)
    be.launch_counts(reset=True)
    h2, h = vectors.run(be, both, 2, x, res, params=p)
    counts = be.launch_counts(reset=True)
    assert np.array_equal(h, h_alone) and np.array_equal(h2, h2_alone)
    assert counts.get("rmsnorm_fused") == 1, counts
    be.trace(2)
    be.trace_reset()
    vectors.run(be, both, 2, x, res, params=p)
    names = set(be.trace_report())
    be.trace(False)
    if shape[:2] in ((512, 8192), (256, 2048), (512, 2048)):  # split along k: the sum is the norm's
        assert any(n.startswith("rmsnorm_fused[") and "k-slices" in n for n in names), sorted(names)


@pytest.mark.parametrize("cfg", [(1, 32, 8, 513, 64), (1, 4, 4, 7, 16), (2, 8, 2, 100, 128), (1, 4, 1, 33, 256),
                                 (1, 16, 16, 1, 64), (1, 2, 1, 9000, 64), (1, 32, 8, 2049, 128),
                                 (3, 4, 2, 700, 256)])  # b, heads, kv heads, T, d
def test_attention_decode(oracle, hip, hip_nopat, cfg):
    """One-query attention over a cache (q . K^T / sqrt(d) + mask, softmax, . V) as one launch."""
    nb, H, KV, T, d = cfg
    g = np.random.default_rng(T * 3 + d)
    q = g.standard_normal((nb, H, 1, d)).astype(np.float32)
    k = g.standard_normal((nb, KV, T, d)).astype(np.float32)
    v = g.standard_normal((nb, KV, T, d)).astype(np.float32)

    def f(b, qv, kv, vv):
        qv, kv, vv = qv + qv - qv, kv + kv - kv, vv + vv - vv      # computed f32 values
        kr = helpers.repeat_kv(b, H // KV, kv)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        attn = attn + lang.broadcast(b, helpers.causal_mask(b, lang.to_nat(b, 1)), sh)
        return lang.matmul(b, nn.softmax(b, attn), vr)
    (ref,) = vectors.run(oracle, f, 1, q, k, v)
    got, names = run_traced(hip, f, 1, q, k, v)
    gen, gnames = run_traced(hip_nopat, f, 1, q, k, v)
    assert "attn_decode" in names and "softmax_fused" not in names, sorted(names)
    assert "attn_decode" not in gnames
    s = np.einsum("bhd,bhtd->bht", q[:, :, 0].astype(np.float64), np.repeat(k, H // KV, 1).astype(np.float64)) / np.sqrt(d)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    expect = np.einsum("bht,bhtd->bhd", p, np.repeat(v, H // KV, 1).astype(np.float64))[:, :, None]
    assert np.allclose(ref, expect, rtol=1e-4, atol=1e-5)
    assert np.allclose(got[0], ref, rtol=1e-4, atol=1e-5), np.abs(got[0] - ref).max()
    assert np.allclose(gen[0], ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("T", [20, 40, 300, 540, 1000, 1500])
@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_attention_decode_merged_by_the_output_projection(oracle, hip, hip_bf16, cg, T, mode):
    """llama.rs:107-112 for one query row: the attention, the head merge (transpose + reshape) and
    `residual + o_proj(.)`.  When the keys are divided over 2 .. 8 workgroups per head the attention launch
    stops at its partial results and the projection's kernel merges them on its way in (a launch named
    ...[attn-merge...]); shorter and longer caches take the attention kernel's own merge.  Either way the
    result is the oracle's."""
    H, KV, d, N = 32, 8, 64, 384
    g = np.random.default_rng(T)
    bf = vectors.bf16_round if mode == "bf16" else (lambda a: a)
    q = g.standard_normal((1, H, 1, d)).astype(np.float32)
    k = g.standard_normal((1, KV, T, d)).astype(np.float32)
    v = g.standard_normal((1, KV, T, d)).astype(np.float32)
    res = g.standard_normal((1, 1, N)).astype(np.float32)
    w = bf((g.standard_normal((N, H * d)) * 0.05).astype(np.float32))
    p = {"o.weight": w}

    def f(b, qv, kv, vv, rv):
        qv, kv, vv, rv = qv + qv - qv, kv + kv - kv, vv + vv - vv, rv + rv - rv
        kr = helpers.repeat_kv(b, H // KV, kv)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        attn = attn + lang.broadcast(b, helpers.causal_mask(b, lang.to_nat(b, 1)), sh)
        out = lang.matmul(b, nn.softmax(b, attn), vr)
        out = lang.reshape(b, lang.make_shape(b, 1, 1, H * d), lang.transpose(b, 1, 2, out))
        return rv + nn.linear_no_bias(b, H * d, N, lang.path(["o"]), out)
    (ref,) = vectors.run(oracle, f, 1, q, k, v, res, params=p)
    be = hip_bf16 if mode == "bf16" else hip
    be.trace(2)
    be.trace_reset()
    (got,) = vectors.run(be, f, 1, q, k, v, res, params=p)
    names = set(be.trace_report())
    be.trace(False)
    assert any(nm.startswith("attn_decode") for nm in names), sorted(names)
    merged = any("attn-merge" in nm for nm in names)
    ns = max(-(-T // 128), min(8, -(-T // 32)))              # the runtime's rule for 32 heads on 256 CUs ...
    if ns <= 8:
        ns = max(-(-T // 110), min(3, -(-T // 32)))          # ... and for key ranges the projection merges
    splits = -(-T // -(-T // ns)) if ns >= 2 else 1
    assert merged == (2 <= splits <= 8), (splits, sorted(names))
    tol = 2e-2 if mode == "bf16" else 1e-4
    assert np.max(np.abs(got - ref)) <= tol * np.abs(ref).max(), np.max(np.abs(got - ref)) / np.abs(ref).max()


def test_attention_decode_merge_needs_the_head_order(oracle, hip, cg):
    """The same chain with a head merge that reorders: `transpose(1, 3)` of [1, H, 1, d] puts d before the
    heads, so the row o_proj reads is (d, head)-ordered.  The projection's merging prologue reads partials in
    (head, d) order and must not take this graph; the result is the oracle's either way."""
    H, KV, d, N, T = 32, 8, 64, 384, 300
    g = np.random.default_rng(77)
    q = g.standard_normal((1, H, 1, d)).astype(np.float32)
    k = g.standard_normal((1, KV, T, d)).astype(np.float32)
    v = g.standard_normal((1, KV, T, d)).astype(np.float32)
    res = g.standard_normal((1, 1, N)).astype(np.float32)
    p = {"o.weight": (g.standard_normal((N, H * d)) * 0.05).astype(np.float32)}

    def f(b, qv, kv, vv, rv):
        qv, kv, vv, rv = qv + qv - qv, kv + kv - kv, vv + vv - vv, rv + rv - rv
        kr = helpers.repeat_kv(b, H // KV, kv)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        attn = attn + lang.broadcast(b, helpers.causal_mask(b, lang.to_nat(b, 1)), sh)
        out = lang.matmul(b, nn.softmax(b, attn), vr)
        out = lang.reshape(b, lang.make_shape(b, 1, 1, H * d), lang.transpose(b, 1, 3, out))   # [1, d, 1, H]
        return rv + nn.linear_no_bias(b, H * d, N, lang.path(["o"]), out)
    (ref,) = vectors.run(oracle, f, 1, q, k, v, res, params=p)
    hip.trace(2)
    hip.trace_reset()
    (got,) = vectors.run(hip, f, 1, q, k, v, res, params=p)
    names = set(hip.trace_report())
    hip.trace(False)
    assert not any("attn-merge" in nm for nm in names), sorted(names)
    assert np.max(np.abs(got - ref)) <= 1e-4 * np.abs(ref).max(), np.max(np.abs(got - ref)) / np.abs(ref).max()


def test_attention_decode_that_cannot_be_fused_still_appends_its_rows(oracle, hip_bf16, cg):
    """A decode step whose caches qualify for the append inside the attention kernel, but whose query
    does not (an uploaded rank-4 tensor is bf16 storage in bf16 mode): the new key and value rows must
    end up in the caches all the same, and the step must give the unfused path's result."""
    H, KV, T0, d = 4, 2, 12, 16
    g = np.random.default_rng(77)
    bf = vectors.bf16_round
    k0, v0 = (bf(g.standard_normal((1, KV, T0, d)).astype(np.float32)) for _ in range(2))
    k1, v1, kn, vn = (bf(g.standard_normal((1, KV, 1, d)).astype(np.float32)) for _ in range(4))
    q = bf(g.standard_normal((1, H, 1, d)).astype(np.float32))

    def grow(b, a, c):                                   # a computed f32 cache with spare rows
        return lang.concat(b, 2, a + a - a, c + c - c)

    def step(b, qv, kc, vc, kx, vx):
        k = lang.concat(b, 2, kc, kx + kx - kx)
        v = lang.concat(b, 2, vc, vx + vx - vx)
        kr, vr = helpers.repeat_kv(b, H // KV, k), helpers.repeat_kv(b, H // KV, v)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        attn = attn + lang.broadcast(b, helpers.causal_mask(b, lang.to_nat(b, 1)), sh)
        return lang.matmul(b, nn.softmax(b, attn), vr), k, v

    res = []
    for be in (oracle, hip_bf16):
        it = cg.Interpreter(be, cg.stdlib())
        gt = vectors.Fn("grow", 2, 1, grow).term()
        (kc,) = it.run(gt, [be.tensor(k0), be.tensor(k1)])
        (vc,) = it.run(gt, [be.tensor(v0), be.tensor(v1)])
        be.realize(kc), be.realize(vc)
        st = vectors.Fn("step", 5, 3, step).term()
        if be is hip_bf16:
            be.trace(True)
            be.trace_reset()
        out, k, v = it.run(st, [be.tensor(q), kc, vc, be.tensor(kn), be.tensor(vn)], moved=(1, 2))
        res.append([be.numpy(out), be.numpy(k), be.numpy(v)])
        if be is hip_bf16:
            names = set(be.trace_report())
            be.trace(False)
            # the rows went in through their own launches, into the caches' own storage
            assert "kv_append" in names and "attn_decode" not in names, sorted(names)
    (ro, rk, rv), (go, gk, gv) = res
    assert np.array_equal(rk, np.concatenate([k0, k1, kn], axis=2)) and np.array_equal(gk, rk)
    assert np.array_equal(gv, rv) and np.array_equal(rv, np.concatenate([v0, v1, vn], axis=2))
    assert np.max(np.abs(go - ro)) <= 2e-2 * np.abs(ro).max()


@pytest.mark.parametrize("K", [2048, 256, 1152])
@pytest.mark.parametrize("variant", ["llama", "gemma", "extra_consumer"])
def test_rmsnorm_in_projection_prologue(oracle, hip, hip_bf16, hip_nopat, K, variant):
    """rmsnorm(x) feeding q/k/v-style one-row projections: the norm runs inside the product launch
    (no rmsnorm launch) unless something else also reads the normed row."""
    g = np.random.default_rng(K)
    x = (g.standard_normal((1, 1, K)) * 2).astype(np.float32)
    p = {"n.weight": g.standard_normal(K).astype(np.float32)}
    outs = [K, 512, 264]
    for i, o in enumerate(outs):
        p[f"l{i}.weight"] = (g.standard_normal((o, K)) * 0.05).astype(np.float32)

    def f(b, xv):
        xv = xv + xv - xv
        if variant == "gemma":
            gm = lang.param(b, lang.path(["n", "weight"]))
            raw = helpers.rmsnorm_raw(b, 1e-6, xv)
            gm = lang.broadcast(b, gm, lang.shape(b, raw))
            h = raw * (lang.constant(b, 1.0, lang.shape(b, gm)) + gm)
        else:
            h = helpers.rmsnorm(b, 1e-5, lang.path(["n"]), xv)
        ys = [nn.linear_no_bias(b, K, o, lang.path([f"l{i}"]), h) for i, o in enumerate(outs)]
        if variant == "extra_consumer":
            ys.append(h + h)
        return ys
    n_out = len(outs) + (variant == "extra_consumer")
    ref = vectors.run(oracle, f, n_out, x, params=p)
    got, names = run_traced(hip, f, n_out, x, params=p)
    gen = vectors.run(hip_nopat, f, n_out, x, params=p)
    if variant == "extra_consumer":
        assert "rmsnorm_fused" in names
    else:
        assert "rmsnorm_fused" not in names and "gemv_rowdot_f32" in names, sorted(names)
    for r, a, c in zip(ref, got, gen):
        assert np.allclose(a, r, rtol=1e-4, atol=1e-5), np.abs(a - r).max()
        assert np.allclose(c, r, rtol=1e-4, atol=1e-5)
    p16 = {k: (vectors.bf16_round(v) if v.ndim >= 2 else v) for k, v in p.items()}
    ref16 = vectors.run(oracle, f, n_out, x, params=p16)
    got16, names16 = run_traced(hip_bf16, f, n_out, x, params=p)
    if variant != "extra_consumer":
        assert "rmsnorm_fused" not in names16 and "gemv_rowdot_bf16" in names16, sorted(names16)
    for r, a in zip(ref16, got16):
        assert np.max(np.abs(a - r)) <= 2e-2 * np.abs(r).max()


@pytest.mark.parametrize("K,N", [(8192, 2048), (512, 96), (6912, 1152)])
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_glu_in_projection_prologue(oracle, hip, hip_nopat, K, N, act):
    """down_proj(silu(gate) * up) + residual as one launch."""
    g = np.random.default_rng(K + N)
    gate = g.standard_normal((1, 1, K)).astype(np.float32)
    up = g.standard_normal((1, 1, K)).astype(np.float32)
    res = g.standard_normal((1, 1, N)).astype(np.float32)
    p = {"d.weight": (g.standard_normal((N, K)) * 0.02).astype(np.float32)}

    def f(b, gv, uv, rv):
        gv, uv = gv + gv - gv, uv + uv - uv
        h = (nn.silu(b, gv) if act == "silu" else nn.gelu(b, gv)) * uv
        return nn.linear_no_bias(b, K, N, lang.path(["d"]), h) + rv
    (ref,) = vectors.run(oracle, f, 1, gate, up, res, params=p)
    got, names = run_traced(hip, f, 1, gate, up, res, params=p)
    (gen,) = vectors.run(hip_nopat, f, 1, gate, up, res, params=p)
    assert not ({"swiglu_fused", "geglu_fused", "binary_f32"} & names), sorted(names)
    assert np.allclose(got[0], ref, rtol=1e-4, atol=1e-5), np.abs(got[0] - ref).max()
    assert np.allclose(gen, ref, rtol=1e-4, atol=1e-5)


def _folded_linear(b, i, o, name, x):
    """A linear over [B, 1, K] the way a batch-correct model writes it: the batch folded into the rows
    of one matrix for the product and unfolded again (catgrad-llm/src/legacy/nn/layers.rs:435-456)."""
    bb, ss, hh = lang.unpack(b, 3, lang.shape(b, x))
    y = nn.linear_no_bias(b, i, o, lang.path([name]), lang.reshape(b, lang.make_shape(b, 1, bb * ss, hh), x))
    return lang.reshape(b, lang.make_shape(b, bb, ss, o), y)


@pytest.mark.parametrize("rows", [1, 3])
def test_biased_projections_of_a_decode_step(oracle, hip, hip_bf16, hip_nopat, rows):
    """q/k/v linears with a bias (Qwen-style attention) on the normed rows of a decode step: one launch
    that computes the norm, the three products and adds each bias vector to every row of its product."""
    K = 512
    g = np.random.default_rng(rows)
    x = (g.standard_normal((rows, 1, K)) * 2).astype(np.float32)
    p = {"n.weight": g.standard_normal(K).astype(np.float32)}
    outs = {"q": K, "k": 128, "v": 192}
    for name, o in outs.items():
        p[name + ".weight"] = (g.standard_normal((o, K)) * 0.05).astype(np.float32)
        p[name + ".bias"] = g.standard_normal(o).astype(np.float32)

    def lin(b, o, name, h):
        bb, ss, hh = lang.unpack(b, 3, lang.shape(b, h))
        y = nn.linear(b, K, o, lang.path([name]), lang.reshape(b, lang.make_shape(b, 1, bb * ss, hh), h))
        return lang.reshape(b, lang.make_shape(b, bb, ss, o), y)

    def f(b, xv):
        xv = xv + xv - xv
        h = helpers.rmsnorm(b, 1e-5, lang.path(["n"]), xv)
        return [lin(b, o, name, h) for name, o in outs.items()]
    ref = vectors.run(oracle, f, 3, x, params=p)
    hip.trace(True)
    hip.trace_reset()
    got = vectors.run(hip, f, 3, x, params=p)
    rep = hip.trace_report()
    hip.trace(False)
    launches = {k: v["launches"] for k, v in rep.items()}
    assert launches == {"ew_fused": 1, "gemv_rowdot_f32": 1}, launches      # x + x - x, then everything else
    gen = vectors.run(hip_nopat, f, 3, x, params=p)
    for r, a, c in zip(ref, got, gen):
        assert a.shape == r.shape and np.allclose(a, r, rtol=1e-4, atol=1e-4), np.abs(a - r).max()
        assert np.allclose(c, r, rtol=1e-4, atol=1e-4)
    p16 = {k: (vectors.bf16_round(v) if v.ndim >= 2 else v) for k, v in p.items()}
    ref16 = vectors.run(oracle, f, 3, x, params=p16)
    got16, names16 = run_traced(hip_bf16, f, 3, x, params=p)
    assert "binary_f32" not in names16 and "rmsnorm_fused" not in names16, sorted(names16)
    for r, a in zip(ref16, got16):
        assert np.max(np.abs(a - r)) <= 2e-2 * np.abs(r).max()


@pytest.mark.parametrize("rows,K,N", [(2, 128, 64), (5, 256, 200), (8, 1152, 1000), (16, 1024, 72), (3, 5632, 2100),
                                      (4, 2048, 2050), (16, 1152, 64), (7, 384, 83), (13, 640, 4099)])
def test_few_rows_on_the_matrix_cores(hip_bf16, rows, K, N):
    """2 to 16 rows against a bf16 weight matrix: the weights go from memory into the MFMA operand and the
    rows are rounded to bf16 on their way into LDS, so the result is the product of the rounded operands,
    accumulated in f32 - checked against exactly that in float64, with and without a residual."""
    g = np.random.default_rng(rows * 100 + K)
    x = g.standard_normal((rows, 1, K)).astype(np.float32)
    res = g.standard_normal((rows, 1, N)).astype(np.float32)
    p = {"w.weight": (g.standard_normal((N, K)) * 0.05).astype(np.float32)}
    want = vectors.bf16_round(x.reshape(rows, K)).astype(np.float64) @ vectors.bf16_round(p["w.weight"]).astype(np.float64).T
    scale = np.abs(want).max()

    def plain(b, xv):
        return _folded_linear(b, K, N, "w", xv + xv - xv)

    def with_residual(b, xv, rv):
        rv = rv + rv - rv   # (arrays of two or more axes are loaded as bf16 in this mode: an f32 value with two readers)
        return rv + _folded_linear(b, K, N, "w", xv + xv - xv), rv
    (got,), names = run_traced(hip_bf16, plain, 1, x, params=p)
    assert "gemv_rows_bf16" in names, sorted(names)
    assert got.shape == (rows, 1, N) and np.max(np.abs(got.reshape(rows, N) - want)) <= 1e-5 * scale
    (got, r16), names = run_traced(hip_bf16, with_residual, 2, x, res, params=p)
    assert "gemv_rows_bf16" in names and (rows > 8 or "binary_f32" not in names), sorted(names)
    assert np.array_equal(r16, vectors.bf16_round(res))
    assert np.max(np.abs(got.reshape(rows, N) - (want + r16.reshape(rows, N)))) <= 1e-5 * (scale + np.abs(res).max())


@pytest.mark.parametrize("b,m,n,k", [(1, 1024, 1024, 1024), (8, 256, 384, 512), (1, 4096, 4104, 256), (2, 192, 200, 128),
                                     (1, 130, 72, 64), (3, 64, 64, 64), (1, 512, 136, 4096)])
def test_product_of_two_activations_reads_the_right_operand_where_it_lies(hip_bf16, b, m, n, k):
    """matmul(x [b, m, k], w [b, k, n]) with both operands as they are stored (ndarray.rs:549-615: any layout): in
    bf16 mode the right operand, k-major, goes from memory into LDS as it lies and reaches the MFMA through the
    transposing LDS read - no transposed copy is made first.  Checked against float64 on the rounded operands."""
    g = np.random.default_rng(b * 1000 + m + n + k)
    x = vectors.bf16_round(g.standard_normal((b, m, k)).astype(np.float32))
    w = vectors.bf16_round(g.standard_normal((b, k, n)).astype(np.float32))
    (got,), names = run_traced(hip_bf16, lambda bb, xv, wv: lang.matmul(bb, xv, wv), 1, x, w)
    assert "gemm_mfma_bf16" in names and "transpose_cast_bf16" not in names, sorted(names)
    want = np.einsum("bmk,bkn->bmn", x.astype(np.float64), w.astype(np.float64))
    assert got.shape == want.shape and np.max(np.abs(got - want)) <= 2e-6 * np.abs(want).max() * np.sqrt(k / 64)


@pytest.mark.parametrize("rows,K,widths", [(4, 2048, (60, 1)), (2, 256, (5, 13, 1, 16)), (16, 1024, (33,))])
def test_narrow_products_of_a_few_rows_share_a_launch(hip_bf16, rows, K, widths):
    """The router and the shared expert's gate of a MoE block (qwen_moe.py: 60 and 1 columns on the same
    rows, each a plain linear over [1, rows, K]): one launch of the matrix-core kernel for up to four
    such products, and no other product launch."""
    g = np.random.default_rng(rows + K)
    x = g.standard_normal((1, rows, K)).astype(np.float32)   # (the block sees the batch folded into the rows)
    p = {f"w{i}.weight": (g.standard_normal((n, K)) * 0.05).astype(np.float32) for i, n in enumerate(widths)}

    def f(b, xv):
        xv = xv + xv - xv
        return [nn.linear_no_bias(b, K, n, lang.path([f"w{i}"]), xv) for i, n in enumerate(widths)]
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    got = vectors.run(hip_bf16, f, len(widths), x, params=p)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    launches = {k: v["launches"] for k, v in rep.items() if k.startswith("gem")}
    assert launches == {"gemv_rows_bf16": 1}, launches
    x16 = vectors.bf16_round(x.reshape(rows, K)).astype(np.float64)
    for i, n in enumerate(widths):
        want = x16 @ vectors.bf16_round(p[f"w{i}.weight"]).astype(np.float64).T
        assert got[i].shape == (1, rows, n)
        assert np.max(np.abs(got[i].reshape(rows, n) - want)) <= 1e-5 * max(np.abs(want).max(), 1.0)


@pytest.mark.parametrize("rows,K,N", [(3, 1152, 520), (16, 1152, 96), (4, 4608, 130)])
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_glu_of_a_few_rows_in_the_prologue_of_the_matrix_core_kernel(oracle, hip_bf16, rows, K, N, act):
    """down_proj over the rows of a small batch when gate and up arrive as tensors: the activation and the
    product are computed on the way into LDS."""
    g = np.random.default_rng(rows + K + len(act))
    gate, up = (g.standard_normal((rows, 1, K)).astype(np.float32) for _ in range(2))
    res = g.standard_normal((rows, 1, N)).astype(np.float32)
    p = {"d.weight": (g.standard_normal((N, K)) * 0.05).astype(np.float32)}

    def f(b, gv, uv, rv):
        gv, uv = gv + gv - gv, uv + uv - uv
        h = (nn.silu(b, gv) if act == "silu" else nn.gelu(b, gv)) * uv
        return _folded_linear(b, K, N, "d", h) + rv
    p16 = {k: vectors.bf16_round(v) for k, v in p.items()}
    (ref,) = vectors.run(oracle, f, 1, gate, up, res, params=p16)
    (got,), names = run_traced(hip_bf16, f, 1, gate, up, res, params=p)
    assert "gemv_rows_bf16" in names and not ({"swiglu_fused", "geglu_fused"} & names), sorted(names)
    assert np.max(np.abs(got - ref)) <= 1e-2 * np.abs(ref).max()


@pytest.mark.parametrize("rows,K,N", [(4, 256, 96), (9, 512, 200)])
def test_few_rows_that_are_a_slice_of_wider_rows(hip_bf16, rows, K, N):
    """The input rows as the left half of rows twice as long (a row stride that is not K), and the weights as
    the left half of a wider matrix: whichever kernel runs, the product of the rounded operands."""
    g = np.random.default_rng(rows + K + N)
    x2 = g.standard_normal((1, rows, 2 * K)).astype(np.float32)
    p = {"w.weight": (g.standard_normal((N, 2 * K)) * 0.05).astype(np.float32)}

    def f(b, xv):
        xv = xv + xv - xv
        xs = lang.slice(b, 2, 0, K, xv)
        w = lang.slice(b, 1, 0, K, lang.param(b, lang.path(["w", "weight"])))
        return nn.linear_no_bias_param(b, K, N, w, xs)
    (got,) = vectors.run(hip_bf16, f, 1, x2, params=p)
    want = vectors.bf16_round(x2[0, :, :K]).astype(np.float64) @ vectors.bf16_round(p["w.weight"][:, :K]).astype(np.float64).T
    assert got.shape == (1, rows, N) and np.max(np.abs(got[0] - want)) <= 1e-5 * np.abs(want).max()


@pytest.mark.parametrize("rows,K", [(17, 256), (16, 2048), (4, 320), (4, 5632)])
def test_rows_the_matrix_core_kernel_does_not_take(oracle, hip_bf16, rows, K):
    """More than 16 rows, rows that do not fit its LDS, K that its four waves cannot split evenly, or a
    deep matrix with too few columns to occupy the CUs: another kernel computes the product, to the
    tolerance of bf16 mode."""
    N = 96
    g = np.random.default_rng(rows + K)
    x = g.standard_normal((rows, 1, K)).astype(np.float32)
    p = {"w.weight": (g.standard_normal((N, K)) * 0.05).astype(np.float32)}

    def f(b, xv):
        return _folded_linear(b, K, N, "w", xv + xv - xv)
    p16 = {k: vectors.bf16_round(v) for k, v in p.items()}
    (ref,) = vectors.run(oracle, f, 1, x, params=p16)
    (got,), names = run_traced(hip_bf16, f, 1, x, params=p)
    assert "gemv_rows_bf16" not in names, sorted(names)
    assert np.max(np.abs(got - ref)) <= 2e-2 * np.abs(ref).max()


@pytest.mark.parametrize("rows,dims", [(2, (512, 1024)), (3, (512, 1024)), (4, (512, 1024)), (4, (640, 1152)), (8, (512, 1024)),
                                       (13, (640, 1152)), (16, (512, 1024)), (16, (640, 1152))])
@pytest.mark.parametrize("act", ["silu", "gelu"])
def test_decoder_block_of_a_small_batch(oracle, hip, hip_bf16, hip_nopat, rows, dims, act):
    """One decode step of `rows` sequences through the projections of a decoder layer, each linear
    folding the batch itself: RMSNorm inside the grouped q/k/v launch, the residual in o_proj's
    epilogue, gate_proj, up_proj and the activation as one launch - five launches where the rows taken
    one product at a time need eleven - and the same values as the oracle.  f32 weights take up to 4 rows
    this way; bf16 weights up to 16, on the matrix cores."""
    K, F = dims
    g = np.random.default_rng(rows * 10 + len(act))
    x = (g.standard_normal((rows, 1, K)) * 2).astype(np.float32)
    p = {"n1.weight": g.standard_normal(K).astype(np.float32), "n2.weight": g.standard_normal(K).astype(np.float32)}
    for name, (o, i) in {"q": (K, K), "k": (128, K), "v": (128, K), "o": (K, K), "g": (F, K), "u": (F, K), "d": (K, F)}.items():
        p[name + ".weight"] = (g.standard_normal((o, i)) * 0.05).astype(np.float32)

    def f(b, xv):
        xv = xv + xv - xv
        h = helpers.rmsnorm(b, 1e-5, lang.path(["n1"]), xv)
        q, k, v = (_folded_linear(b, K, o, nm, h) for nm, o in (("q", K), ("k", 128), ("v", 128)))
        xv = xv + _folded_linear(b, K, K, "o", q)        # (attention itself is not part of this test)
        h = helpers.rmsnorm(b, 1e-5, lang.path(["n2"]), xv)
        gt, up = _folded_linear(b, K, F, "g", h), _folded_linear(b, K, F, "u", h)
        m = (nn.silu(b, gt) if act == "silu" else nn.gelu(b, gt)) * up
        return xv + _folded_linear(b, F, K, "d", m), k, v
    ref = vectors.run(oracle, f, 3, x, params=p)
    got, names = run_traced(hip, f, 3, x, params=p)
    gen = vectors.run(hip_nopat, f, 3, x, params=p)
    if rows <= 4:
        assert not ({"rmsnorm_fused", "swiglu_fused", "geglu_fused", "binary_f32"} & names), sorted(names)
    hip.trace(True)
    hip.trace_reset()
    vectors.run(hip, f, 3, x, params=p)
    rep = hip.trace_report()
    hip.trace(False)
    # x + x - x, then q/k/v, o_proj, gate/up, down_proj
    if rows <= 4:
        assert rep["gemv_rowdot_f32"]["launches"] == 4 and sum(v["launches"] for v in rep.values()) == 5, {k: v["launches"] for k, v in rep.items()}
    for r, a, c in zip(ref, got, gen):
        assert a.shape == r.shape and np.allclose(a, r, rtol=1e-4, atol=1e-4), np.abs(a - r).max()
        assert np.allclose(c, r, rtol=1e-4, atol=1e-4)
    p16 = {k: (vectors.bf16_round(v) if v.ndim >= 2 else v) for k, v in p.items()}
    ref16 = vectors.run(oracle, f, 3, x, params=p16)
    got16, names16 = run_traced(hip_bf16, f, 3, x, params=p)
    if rows <= 8:   # (a residual rides in the epilogue for up to 8 rows)
        assert not ({"rmsnorm_fused", "swiglu_fused", "geglu_fused", "binary_f32"} & names16), sorted(names16)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    vectors.run(hip_bf16, f, 3, x, params=p)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    assert rep["gemv_rows_bf16"]["launches"] == 4, {k: v["launches"] for k, v in rep.items()}
    for r, a in zip(ref16, got16):
        assert np.max(np.abs(a - r)) <= 2e-2 * np.abs(r).max()


@pytest.mark.parametrize("K,N", [(2048, 128256), (2048, 4100), (512, 9001), (4096, 40000), (8192, 4096), (2048, 4095)])
@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_argmax_of_the_row_a_projection_stores(oracle, hip, hip_bf16, hip_nopat, K, N, mode):
    """Greedy decoding: final norm, lm_head, argmax over the logits.  The product's launch keeps the largest
    value each wave stores and the argmax merges those records (one small launch) instead of reading the row
    back.  Equal maxima: the last one wins, as in the reference (ndarray.rs:469-480) - the matrix holds the same
    row several times.  Same index as the op-at-a-time evaluation of the same logits."""
    be = hip if mode == "f32" else hip_bf16
    g = np.random.default_rng(K + N)
    x = g.standard_normal((1, 1, K)).astype(np.float32)
    w = vectors.bf16_round((g.standard_normal((N, K)) * 0.05).astype(np.float32))
    p = {"n.weight": g.standard_normal(K).astype(np.float32), "l.weight": w}

    def f(b, xv):
        xv = xv + xv - xv      # a computed f32 row, like the residual stream
        lg = nn.linear_no_bias(b, K, N, lang.path(["l"]), helpers.rmsnorm(b, 1e-5, lang.path(["n"]), xv))
        return lang.argmax(b, lg), lg
    tok, lg = vectors.run(be, f, 2, x, params=p)
    # the winning row three more times, one of them in the last column: four equal maxima
    top = int(np.argmax(lg.reshape(-1)))
    for at in (7, N // 2 + 1, N - 1):
        w[at] = w[top]
    be.launch_counts(reset=True)
    tok, lg = vectors.run(be, f, 2, x, params=p)
    counts = be.launch_counts(reset=True)
    flat = lg.reshape(-1)
    assert flat[7] == flat[top] == flat[N - 1] == flat.max()
    assert int(tok.reshape(-1)[0]) == N - 1
    for other in (hip_nopat, oracle):   # the argmax op on its own, over the same logits
        (alone,) = vectors.run(other, lambda b, v: lang.argmax(b, v), 1, lg.reshape(-1))
        assert int(np.asarray(alone).reshape(-1)[0]) == N - 1
    x16 = vectors.bf16_round(x) if mode == "bf16" else x
    ref_tok, ref_lg = vectors.run(oracle, f, 2, x16, params=p)
    assert np.max(np.abs(lg - ref_lg)) <= (1e-4 if mode == "f32" else 2e-2) * np.abs(ref_lg).max()
    counts.pop("ew_to_bf16", None)   # (the parameters on their way in)
    assert counts.get("reduce_argmax") == 1 and sum(counts.values()) == 3, counts   # x + x - x, product, argmax
    be.trace(2)
    be.trace_reset()
    vectors.run(be, f, 2, x, params=p)
    names = set(be.trace_report())
    be.trace(False)
    # the one-row kernel leaves the records unless it splits k over its waves (deep and narrow: (8192, 4096)):
    # the argmax reads those, not the row
    assert ("reduce_argmax[records]" in names) == (N >= 4096 and (K, N) != (8192, 4096)), sorted(names)


@pytest.mark.parametrize("rows,d,k", [(4, 2048, 4), (2, 64, 2), (37, 260, 6), (3, 8, 1)])
def test_sum_of_rows_scaled_by_their_own_values(oracle, hip, hip_nopat, rows, d, k):
    """How a MoE block ends (llm/qwen_moe.py): the k expert rows times their router values, summed from zero
    in a [rows, 1, d] frame, transposed to [1, rows, d], plus the shared expert's rows through a sigmoid gate,
    unfolded to [rows, 1, d], plus the residual - one launch, and the bits of the one-op-at-a-time evaluation
    on the same device (every product and sum rounded on its own, in the same order; the oracle's exp differs
    from the device's in the last place)."""
    g = np.random.default_rng(rows * 7 + d + k)
    hs = [g.standard_normal((rows, 1, d)).astype(np.float32) for _ in range(k)]
    vals = g.random((rows, k)).astype(np.float32)
    shared = g.standard_normal((1, rows, d)).astype(np.float32)
    gate = g.standard_normal((1, rows, 1)).astype(np.float32)
    res = g.standard_normal((rows, 1, d)).astype(np.float32)

    def f(b, *a):
        h, (v, sh, gt, rs) = a[:k], a[k:]
        acc = lang.constant(b, 0.0, lang.shape(b, h[0]))
        for i in range(k):
            vi = helpers.unsqueeze(b, 2, 2, lang.get(b, 1, i, v))
            acc = acc + h[i] * lang.broadcast(b, vi, lang.shape(b, h[i]))
        acc = lang.transpose(b, 0, 1, acc)
        out = acc + sh * lang.broadcast(b, nn.sigmoid(b, gt), lang.shape(b, sh))
        out = lang.reshape(b, lang.shape(b, rs), out)
        return out + rs
    args = (*hs, vals, shared, gate, res)
    (ref,) = vectors.run(oracle, f, 1, *args)
    (got,), names = run_traced(hip, f, 1, *args)
    (gen,) = vectors.run(hip_nopat, f, 1, *args)
    assert names == {"row_scaled_sum"}, sorted(names)
    assert got.shape == ref.shape and np.array_equal(got, gen), np.abs(got - gen).max()
    assert np.allclose(got, ref, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("variant", ["right_nested", "shared_term", "two_chains", "scale_on_the_left", "nine_terms"])
def test_sum_of_scaled_rows_in_other_arrangements(hip, hip_nopat, variant):
    """Additions nested to the right, a term somebody else reads too, two chains under one addition, the scale as
    the left factor, more terms than the kernel takes: whatever part the row kernel computes, the values are
    those of the one-op-at-a-time evaluation, bit for bit."""
    rows, d = 5, 128
    g = np.random.default_rng(len(variant))
    xs = [g.standard_normal((rows, 1, d)).astype(np.float32) for _ in range(9)]
    sc = [g.random((rows, 1, 1)).astype(np.float32) for _ in range(3)]

    def f(b, *a):
        x, s = a[:9], [lang.broadcast(b, v, lang.shape(b, a[0])) for v in a[9:]]
        if variant == "right_nested":
            return [x[0] + (x[1] * s[0] + (x[2] + x[3] * s[1]))]
        if variant == "shared_term":
            t = x[1] * s[0]
            return [x[0] + t + x[2] * s[1], t + x[3]]
        if variant == "two_chains":
            return [(x[0] + x[1] * s[0] + x[2]) + (x[3] * s[1] + x[4] + x[5] * s[2])]
        if variant == "scale_on_the_left":
            return [s[0] * x[0] + s[1] * x[1] + x[2]]
        out = x[0] * s[0]
        for i in range(1, 9):
            out = out + x[i] * s[i % 3]
        return [out]
    n_out = 2 if variant == "shared_term" else 1
    got = vectors.run(hip, f, n_out, *xs, *sc)
    gen = vectors.run(hip_nopat, f, n_out, *xs, *sc)
    for a, c in zip(got, gen):
        assert a.shape == c.shape and np.array_equal(a, c), np.abs(a - c).max()


def test_sums_the_row_kernel_leaves_alone(oracle, hip):
    """Two terms, no scale, or a scale that is not one value per row: the usual kernels."""
    g = np.random.default_rng(5)
    a, b_, c = (g.standard_normal((3, 1, 64)).astype(np.float32) for _ in range(3))
    col = g.standard_normal((1, 1, 64)).astype(np.float32)

    def plain(b, x, y, z):
        return x + y + z

    def by_column(b, x, y, z, w):
        return x + y + z * lang.broadcast(b, w, lang.shape(b, z))
    (ref,) = vectors.run(oracle, plain, 1, a, b_, c)
    (got,), names = run_traced(hip, plain, 1, a, b_, c)
    assert "row_scaled_sum" not in names and np.array_equal(got, ref)
    (ref,) = vectors.run(oracle, by_column, 1, a, b_, c, col)
    (got,), names = run_traced(hip, by_column, 1, a, b_, c, col)
    assert "row_scaled_sum" not in names and np.allclose(got, ref, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("order", ["res_first", "norm_first"])
@pytest.mark.parametrize("shape", [(2, 33, 1152), (1, 7, 64)])
def test_rmsnorm_plus_residual(oracle, hip, hip_nopat, shape, order):
    """gemma3.rs:198-240: res + rmsnorm(x) (1 + gamma form) in the RMSNorm kernel."""
    g = np.random.default_rng(shape[1])
    x = (g.standard_normal(shape) * 2).astype(np.float32)
    res = g.standard_normal(shape).astype(np.float32)
    p = {"n.weight": (g.standard_normal(shape[-1]) * 0.1).astype(np.float32)}

    def f(b, xv, rv):
        xv = xv + xv - xv           # the residual stream is a value in memory; the normed branch is computed
        gm = lang.param(b, lang.path(["n", "weight"]))
        raw = helpers.rmsnorm_raw(b, 1e-6, xv)
        gm = lang.broadcast(b, gm, lang.shape(b, raw))
        h = raw * (lang.constant(b, 1.0, lang.shape(b, gm)) + gm)
        return rv + h if order == "res_first" else h + rv
    check(oracle, hip, hip_nopat, f, 1, [x, res], "rmsnorm_fused", params=p, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", [(2, 33, 1152), (1, 40, 64), (4, 64, 256), (1, 7, 64), (1, 2050, 1152), (2, 1027, 640)])
def test_two_norms_around_a_residual_add(oracle, hip, hip_bf16, hip_nopat, shape):
    """gemma3.rs:198-240: `mid = res + norm(y)` and right after it `norm(mid)` (post-attention and
    pre-feedforward norms; post-feedforward and the next layer's input norm).  With many rows one
    launch writes mid and norms it again; a later reader of mid (the next residual add) finds it in
    memory."""
    g = np.random.default_rng(shape[1] + shape[2])
    y = (g.standard_normal(shape) * 2).astype(np.float32)
    res = g.standard_normal(shape).astype(np.float32)
    p = {"a.weight": (g.standard_normal(shape[-1]) * 0.1).astype(np.float32),
         "b.weight": (g.standard_normal(shape[-1]) * 0.1).astype(np.float32)}

    def gemma_norm(b, name, v):
        gm = lang.param(b, lang.path([name, "weight"]))
        raw = helpers.rmsnorm_raw(b, 1e-6, v)
        gm = lang.broadcast(b, gm, lang.shape(b, raw))
        return raw * (lang.constant(b, 1.0, lang.shape(b, gm)) + gm)

    def f(b, yv, rv):
        yv = yv + yv - yv
        mid = rv + gemma_norm(b, "a", yv)
        h = gemma_norm(b, "b", mid)
        return h, mid + h
    ref = vectors.run(oracle, f, 2, y, res, params=p)
    hip.trace(True)
    hip.trace_reset()
    got = vectors.run(hip, f, 2, y, res, params=p)
    rep = hip.trace_report()
    hip.trace(False)
    gen = vectors.run(hip_nopat, f, 2, y, res, params=p)
    many = shape[0] * shape[1] >= 32
    assert rep["rmsnorm_fused"]["launches"] == (1 if many else 2), {k: v["launches"] for k, v in rep.items()}
    for r, a, c in zip(ref, got, gen):
        assert np.allclose(a, r, rtol=1e-4, atol=1e-5), np.abs(a - r).max()
        assert np.allclose(c, r, rtol=1e-4, atol=1e-5)
    got16 = vectors.run(hip_bf16, f, 2, vectors.bf16_round(y), vectors.bf16_round(res), params=p)
    ref16 = vectors.run(oracle, f, 2, vectors.bf16_round(y), vectors.bf16_round(res), params=p)
    for r, a in zip(ref16, got16):
        assert np.max(np.abs(a - r)) <= 2e-2 * np.abs(r).max()


@pytest.fixture(scope="module")
def hip_bf16_flash():
    """bf16 mode with the one-pass attention kernel enabled for every length."""
    import importlib
    cg = importlib.import_module("catgrad-rs_amd")
    return cg.Backend(cg.load_library(), flags=cg.abi.FLAG_BF16 | cg.abi.FLAG_ATTN_ONE_PASS)


@pytest.fixture(scope="module")
def hip_f32_flash():
    """f32 mode with the one-pass attention kernel enabled for every length."""
    import importlib
    cg = importlib.import_module("catgrad-rs_amd")
    return cg.Backend(cg.load_library(), flags=cg.abi.FLAG_ATTN_ONE_PASS)


@pytest.mark.parametrize("mode", ["bf16", "f32"])
def test_attention_prefill_with_an_arbitrary_shared_mask(oracle, hip_bf16_flash, hip_f32_flash, mode):
    """One [S, T] mask for every batch and head, given as data: its key tiles are classified once
    (all masked: skipped unfetched; all zero: computed without reading the mask; mixed) and the kernel
    must give the oracle's values for each kind - including rows that see no key at all, which the
    reference turns into the mean of V."""
    nb, H, KV, S, d = 2, 4, 2, 384, 64
    g = np.random.default_rng(77)
    q = g.standard_normal((nb, H, S, d)).astype(np.float32)
    k = g.standard_normal((nb, KV, S, d)).astype(np.float32)
    v = g.standard_normal((nb, KV, S, d)).astype(np.float32)
    lo = np.finfo(np.float32).min
    mask = np.where(g.random((S, S)) < 0.5, lo, 0.0).astype(np.float32)      # mixed everywhere ...
    mask[:128, 128:] = lo                                                    # ... except dead tiles,
    mask[128:256, :192] = 0.0                                                # all-zero tiles,
    mask[300:303, :] = lo                                                    # rows that see nothing,
    mask[256:, 64:128] = lo                                                  # and a dead column of tiles in the middle
    mask = mask.reshape(-1)      # uploaded as rank 1 (a value, kept f32 in bf16 mode) and shaped in the graph

    def f(b, qv, kv, vv, mv):
        qv, kv, vv = qv + qv - qv, kv + kv - kv, vv + vv - vv
        mv = lang.reshape(b, lang.make_shape(b, 1, 1, S, S), mv)
        kr = helpers.repeat_kv(b, H // KV, kv)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        attn = attn + lang.broadcast(b, mv, sh)
        return lang.matmul(b, nn.softmax(b, attn), vr)
    (ref,) = vectors.run(oracle, f, 1, q, k, v, mask)
    be, bar = (hip_bf16_flash, 2e-2) if mode == "bf16" else (hip_f32_flash, 1e-4)
    got, names = run_traced(be, f, 1, q, k, v, mask)
    assert "attn_prefill" in names and "attn_mask_tiles" in names and "softmax_fused" not in names, sorted(names)
    scale = np.abs(ref).max()
    assert np.max(np.abs(got[0] - ref)) <= bar * scale, np.max(np.abs(got[0] - ref)) / scale
    # the rows that see nothing: the mean of V, for every head
    assert np.max(np.abs(got[0][:, :, 300:303] - np.repeat(v, H // KV, axis=1).mean(axis=2, keepdims=True))) <= bar * scale


@pytest.mark.parametrize("cfg", [(1, 32, 8, 512, 64), (2, 4, 2, 100, 128), (2, 4, 2, 104, 128), (1, 4, 1, 200, 256),
                                 (1, 8, 8, 33, 64), (1, 2, 1, 1024, 64),
                                 (1, 4, 1, 2048, 256)])  # the last: Gemma-3's heads at its prompt length, window 512
@pytest.mark.parametrize("mask_kind", ["causal", "window"])
def test_attention_prefill_bf16(oracle, hip_bf16_flash, hip_bf16, hip_nopat, cfg, mask_kind):
    """Attention over many query rows in bf16 mode: one launch with online softmax, scores never
    stored; against the oracle (f32) at the bf16 bar and against the generic f32 path."""
    import importlib
    gemma3 = importlib.import_module("catgrad-rs_amd.llm.gemma3")
    nb, H, KV, S, d = cfg
    g = np.random.default_rng(S + d)
    q = g.standard_normal((nb, H, S, d)).astype(np.float32)
    k = g.standard_normal((nb, KV, S, d)).astype(np.float32)
    v = g.standard_normal((nb, KV, S, d)).astype(np.float32)
    model = gemma3.Gemma3Model(importlib.import_module("catgrad-rs_amd.llm").Config(), S)

    def f(b, qv, kv, vv):
        qv, kv, vv = qv + qv - qv, kv + kv - kv, vv + vv - vv      # computed f32 values
        kr = helpers.repeat_kv(b, H // KV, kv)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        n = lang.to_nat(b, S)
        mask = helpers.causal_mask(b, n) if mask_kind == "causal" else model.window_mask(b, n, 512 if S >= 2048 else 17)
        attn = attn + lang.broadcast(b, mask, sh)
        return lang.matmul(b, nn.softmax(b, attn), vr)
    (ref,) = vectors.run(oracle, f, 1, q, k, v)
    got, names = run_traced(hip_bf16_flash, f, 1, q, k, v)
    (gen,) = vectors.run(hip_nopat, f, 1, q, k, v)
    _, default_names = run_traced(hip_bf16, f, 1, q, k, v)
    assert ("attn_prefill" in default_names) == (S >= 512)
    if S % 8 == 0:
        assert "attn_prefill" in names and "softmax_fused" not in names, sorted(names)
    else:       # mask rows and value columns are read 16 bytes at a time: other lengths take the three-launch path
        assert "attn_prefill" not in names
    scale = np.abs(ref).max()
    assert np.max(np.abs(got[0] - ref)) <= 2e-2 * scale, np.max(np.abs(got[0] - ref)) / scale
    assert np.max(np.abs(gen - ref)) <= 1e-4 * scale


@pytest.mark.parametrize("cfg", [(1, 32, 8, 512, 64), (2, 4, 2, 100, 128), (2, 4, 2, 104, 128), (1, 4, 1, 200, 256),
                                 (1, 8, 8, 40, 64), (1, 2, 1, 1024, 64), (1, 8, 2, 320, 128), (2, 2, 2, 72, 256),
                                 (1, 4, 1, 2048, 256)])  # the last: Gemma-3's heads at its prompt length, window 512
@pytest.mark.parametrize("mask_kind", ["causal", "window", "none"])
def test_attention_prefill_f32(oracle, hip_f32_flash, hip, cfg, mask_kind):
    """Attention over many query rows without the bf16 flag: the same single launch with every product
    in f32, against the oracle at the f32 bar (values relative to the largest of the result)."""
    import importlib
    gemma3 = importlib.import_module("catgrad-rs_amd.llm.gemma3")
    nb, H, KV, S, d = cfg
    g = np.random.default_rng(S + d + 1)
    q = g.standard_normal((nb, H, S, d)).astype(np.float32)
    k = g.standard_normal((nb, KV, S, d)).astype(np.float32)
    v = g.standard_normal((nb, KV, S, d)).astype(np.float32)
    model = gemma3.Gemma3Model(importlib.import_module("catgrad-rs_amd.llm").Config(), S)

    def f(b, qv, kv, vv):
        qv, kv, vv = qv + qv - qv, kv + kv - kv, vv + vv - vv
        kr = helpers.repeat_kv(b, H // KV, kv)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qv, lang.transpose(b, 2, 3, kr))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        if mask_kind != "none":
            n = lang.to_nat(b, S)
            mask = helpers.causal_mask(b, n) if mask_kind == "causal" else model.window_mask(b, n, 512 if S >= 2048 else 17)
            attn = attn + lang.broadcast(b, mask, sh)
        return lang.matmul(b, nn.softmax(b, attn), vr)
    (ref,) = vectors.run(oracle, f, 1, q, k, v)
    got, names = run_traced(hip_f32_flash, f, 1, q, k, v)
    _, default_names = run_traced(hip, f, 1, q, k, v)
    assert ("attn_prefill" in default_names) == (S >= 512)
    if S % 8 == 0:
        assert "attn_prefill" in names and "softmax_fused" not in names, sorted(names)
    else:       # mask rows are read 16 bytes at a time: other lengths take the three-launch path
        assert "attn_prefill" not in names
    scale = np.abs(ref).max()
    assert np.max(np.abs(got[0] - ref)) <= 1e-4 * scale, np.max(np.abs(got[0] - ref)) / scale


def test_queries_and_keys_rotated_by_one_launch(oracle, hip_bf16_flash, cg):
    """A prefill attention whose queries and keys both come straight from apply_rope_embedding: one
    launch rotates both (and the rotated keys, a result of the term, are the oracle's)."""
    nb, H, KV, S, d = 1, 4, 2, 96, 64
    g = np.random.default_rng(123)
    # values bf16 storage keeps exactly: the oracle then rotates the same numbers
    q = vectors.bf16_round(g.standard_normal((nb, H, S, d)).astype(np.float32))
    k = vectors.bf16_round(g.standard_normal((nb, KV, S, d)).astype(np.float32))
    v = vectors.bf16_round(g.standard_normal((nb, KV, S, d)).astype(np.float32))
    llm = __import__("importlib").import_module("catgrad-rs_amd.llm")
    cfg = llm.Config(hidden_size=H * d, num_attention_heads=H, num_key_value_heads=KV, rope_theta=10000.0)

    def f(b, qv, kv, vv):
        qv, kv, vv = qv + qv - qv, kv + kv - kv, vv + vv - vv
        cache = helpers.Cache.init(b, cfg, S)
        qr = helpers.apply_rope_embedding(b, 0, d, cache.cos, cache.sin, qv)
        kr = helpers.apply_rope_embedding(b, 0, d, cache.cos, cache.sin, kv)
        kk = helpers.repeat_kv(b, H // KV, kr)
        vr = helpers.repeat_kv(b, H // KV, vv)
        attn = lang.matmul(b, qr, lang.transpose(b, 2, 3, kk))
        sh = lang.shape(b, attn)
        attn = attn / lang.constant(b, float(np.sqrt(np.float32(d))), sh)
        attn = attn + lang.broadcast(b, helpers.causal_mask(b, lang.to_nat(b, S)), sh)
        return lang.matmul(b, nn.softmax(b, attn), vr), kr
    ref = vectors.run(oracle, f, 2, q, k, v)
    hip_bf16_flash.launch_counts(reset=True)
    got = vectors.run(hip_bf16_flash, f, 2, q, k, v)
    counts = hip_bf16_flash.launch_counts(reset=True)
    assert counts.get("rope_fused") == 1 and counts.get("attn_prefill") == 1, counts
    assert np.allclose(got[1], ref[1], rtol=1e-4, atol=1e-5)                 # the rotated keys
    assert np.max(np.abs(got[0] - ref[0])) <= 2e-2 * np.abs(ref[0]).max()

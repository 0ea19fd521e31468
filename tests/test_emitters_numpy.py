"""The graph emitters (`llm/helpers.py`, `llm/llama.py`, `llm/gemma3.py`) against a float64 numpy
statement of the same models written from the reference's sources, not from the emitters:
half-split RoPE with its theta tables (catgrad-llm/src/helpers.rs:164-221), repeat-interleave GQA
(helpers.rs:147-161), causal softmax attention and the Llama layer (models/llama.rs:77-147), the
tiny Llama forward (models/llama.rs:150-204), and Gemma-3's layer: QK-norm, (1 + gamma), sqrt(H)
embedding scale, local / global theta (models/gemma3.rs:41-68, 153-186, 198-292).  The oracle runs
the emitted terms; the numpy code never touches the term builder.  CPU only."""
import numpy as np

import llama_util as U
import model_util as MU
import vectors

cg, llm = U.cg, U.llm
lang = vectors.lang

RTOL = 1e-5  # f32 evaluation of a tiny model against float64


def rel(ref, got):
    r = np.asarray(ref, np.float64).reshape(-1, np.asarray(ref).shape[-1])
    g = np.asarray(got, np.float64).reshape(r.shape)
    floor = np.sqrt(np.mean(r * r, axis=1, keepdims=True))
    return float(np.max(np.abs(r - g) / np.maximum(np.abs(r), floor)))


# ---- the numpy statement ---------------------------------------------------------------------
def np_rope_tables(theta, n, d):
    """helpers.rs:164-193: inv_freq_i = 1 / theta^(2 i / d); angle = pos * inv_freq; both halves alike."""
    i = np.arange(d // 2, dtype=np.float64)
    inv = 1.0 / np.float64(theta) ** (2.0 * i / d)
    ang = np.arange(n, dtype=np.float64)[:, None] * inv[None, :]
    return np.concatenate([np.cos(ang)] * 2, axis=1), np.concatenate([np.sin(ang)] * 2, axis=1)


def np_rope(x, cos, sin, pos):
    """helpers.rs:195-221 on x[..., s, d]: cos * x + sin * (-x_hi, x_lo), positions pos .. pos + s."""
    s, d = x.shape[-2:]
    c, sn = cos[pos:pos + s], sin[pos:pos + s]
    rot = np.concatenate([-x[..., d // 2:], x[..., :d // 2]], axis=-1)
    return c * x + sn * rot


def np_repeat_kv(x, rep):
    """helpers.rs:147-161: head h of the result is kv head h // rep (repeat-interleave)."""
    return np.repeat(x, rep, axis=-3)


def np_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def np_softmax(a):
    e = np.exp(a - a.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def np_attention(q, k, v, first_pos, window=0):
    """q [.., heads, s, d] at positions first_pos .., k and v [.., heads, t, d] at positions 0 ..:
    softmax(q k^T / sqrt(d) + mask) v with mask = f32::MIN where key > query (llama.rs:95-108) or,
    window > 0, query - key >= window."""
    s, t, d = q.shape[-2], k.shape[-2], q.shape[-1]
    a = q @ np.swapaxes(k, -1, -2) / np.sqrt(np.float64(d))
    qi = first_pos + np.arange(s)[:, None]
    kj = np.arange(t)[None, :]
    dead = kj > qi
    if window:
        dead = dead | (qi - kj >= window)
    a = a + np.where(dead, np.float64(np.finfo(np.float32).min), 0.0)
    return np_softmax(a) @ v


def f64(P, name):
    return P[name].astype(np.float64)


def np_llama_logits(cfg, P, ids):
    """Logits of every position of one sequence, models/llama.rs:37-204."""
    H, heads, kvh = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads
    d, rep, S = H // heads, heads // kvh, len(ids)
    cos, sin = np_rope_tables(cfg.rope_theta, S, d)
    E = f64(P, "llama.model.embed_tokens.weight")
    x = E[np.asarray(ids)]
    silu = lambda a: a / (1 + np.exp(-a))
    for l in range(cfg.num_hidden_layers):
        p = f"llama.model.layers.{l}."
        h = np_rms(x, cfg.rms_norm_eps) * f64(P, p + "input_layernorm.weight")
        q = (h @ f64(P, p + "self_attn.q_proj.weight").T).reshape(S, heads, d).transpose(1, 0, 2)
        k = (h @ f64(P, p + "self_attn.k_proj.weight").T).reshape(S, kvh, d).transpose(1, 0, 2)
        v = (h @ f64(P, p + "self_attn.v_proj.weight").T).reshape(S, kvh, d).transpose(1, 0, 2)
        q, k = np_rope(q, cos, sin, 0), np_rope(np_repeat_kv(k, rep), cos, sin, 0)
        a = np_attention(q, k, np_repeat_kv(v, rep), 0)
        a = a.transpose(1, 0, 2).reshape(S, H) @ f64(P, p + "self_attn.o_proj.weight").T
        x = x + a
        h = np_rms(x, cfg.rms_norm_eps) * f64(P, p + "post_attention_layernorm.weight")
        m = silu(h @ f64(P, p + "mlp.gate_proj.weight").T) * (h @ f64(P, p + "mlp.up_proj.weight").T)
        x = x + m @ f64(P, p + "mlp.down_proj.weight").T
    x = np_rms(x, cfg.rms_norm_eps) * f64(P, "llama.model.norm.weight")
    head = E if cfg.tie_word_embeddings else f64(P, "llama.lm_head.weight")
    return x @ head.T


def np_gemma_logits(cfg, P, ids):
    """ids [b, s] -> logits [b, s, V], models/gemma3.rs:41-292 plus the sliding window of the local layers."""
    H, heads, kvh, d = cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    rep = heads // kvh
    ids = np.asarray(ids)
    B, S = ids.shape
    gnorm = lambda x, w: np_rms(x, cfg.rms_norm_eps) * (1.0 + w)
    gelu = lambda a: 0.5 * a * (1 + np.tanh(np.sqrt(2 / np.pi) * (a + 0.044715 * a ** 3)))
    E = f64(P, "gemma3.model.embed_tokens.weight")
    x = E[ids] * np.float64(np.sqrt(np.float32(H)))
    for l in range(cfg.num_hidden_layers):
        p = f"gemma3.model.layers.{l}."
        local = (l + 1) % cfg.sliding_window_pattern != 0
        cos, sin = np_rope_tables(cfg.rope_local_base_freq if local else cfg.rope_theta, S, d)
        res = x
        h = gnorm(x, f64(P, p + "input_layernorm.weight"))
        q = (h @ f64(P, p + "self_attn.q_proj.weight").T).reshape(B, S, heads, d).transpose(0, 2, 1, 3)
        k = (h @ f64(P, p + "self_attn.k_proj.weight").T).reshape(B, S, kvh, d).transpose(0, 2, 1, 3)
        v = (h @ f64(P, p + "self_attn.v_proj.weight").T).reshape(B, S, kvh, d).transpose(0, 2, 1, 3)
        q = np_rope(gnorm(q, f64(P, p + "self_attn.q_norm.weight")), cos, sin, 0)
        k = np_rope(gnorm(k, f64(P, p + "self_attn.k_norm.weight")), cos, sin, 0)
        a = np_attention(q, np_repeat_kv(k, rep), np_repeat_kv(v, rep), 0,
                         cfg.sliding_window if local else 0)
        a = a.transpose(0, 2, 1, 3).reshape(B, S, heads * d) @ f64(P, p + "self_attn.o_proj.weight").T
        x = res + gnorm(a, f64(P, p + "post_attention_layernorm.weight"))
        res = x
        h = gnorm(x, f64(P, p + "pre_feedforward_layernorm.weight"))
        m = gelu(h @ f64(P, p + "mlp.gate_proj.weight").T) * (h @ f64(P, p + "mlp.up_proj.weight").T)
        m = m @ f64(P, p + "mlp.down_proj.weight").T
        x = gnorm(m, f64(P, p + "post_feedforward_layernorm.weight")) + res
    return gnorm(x, f64(P, "gemma3.model.norm.weight")) @ E.T


# ---- the emitted terms on the oracle against it ------------------------------------------------
def test_rope_tables_and_rotation(oracle):
    d, n, theta = 16, 11, 500000.0
    cos, sin = vectors.run(oracle, lambda b: list(llm.helpers.rope_tables(b, theta, lang.to_nat(b, n), d)), 2)
    rc, rs = np_rope_tables(theta, n, d)
    assert np.allclose(cos, rc, rtol=0, atol=2e-6) and np.allclose(sin, rs, rtol=0, atol=2e-6)
    x = np.random.default_rng(0).standard_normal((1, 3, 4, d)).astype(np.float32)
    for pos in (0, 5):
        (y,) = vectors.run(oracle, lambda b, v: llm.helpers.rope(b, theta, pos, 4, d, v), 1, x)
        ref = np_rope(x.astype(np.float64), *np_rope_tables(theta, pos + 4, d), pos)
        assert rel(ref, y) <= RTOL
    # a dropped sign or swapped halves in rotate_half would pass neither: rotation keeps pair norms
    (y,) = vectors.run(oracle, lambda b, v: llm.helpers.rope(b, theta, 3, 4, d, v), 1, x)
    assert np.allclose(y[..., :d // 2] ** 2 + y[..., d // 2:] ** 2, x[..., :d // 2] ** 2 + x[..., d // 2:] ** 2, rtol=1e-5)


def test_repeat_kv_is_repeat_interleave(oracle):
    """Head h of the result is kv head h // rep: numpy's repeat along the head axis, not a tiling."""
    x = np.random.default_rng(1).standard_normal((2, 3, 5, 4)).astype(np.float32)
    (y,) = vectors.run(oracle, lambda b, v: llm.helpers.repeat_kv(b, 4, v), 1, x)
    assert y.shape == (2, 12, 5, 4)
    assert np.array_equal(y, np.repeat(x, 4, axis=1))
    assert not np.array_equal(y, np.tile(x, (1, 4, 1, 1)))  # tiling the heads is the plausible mistake


def test_llama_forward_matches_numpy(oracle):
    """Prefill logits and three KV-cached decode steps of the emitted terms = the last row of the numpy
    forward over the sequence so far (GQA with rep 2, tied head)."""
    cfg = U.tiny_config(num_hidden_layers=2)
    P = U.param_arrays(cfg, seed=11, std=0.2)
    for k in P:
        if k.endswith("layernorm.weight") or k.endswith("model.norm.weight"):
            P[k] = (1.0 + 0.1 * np.random.default_rng(len(k)).standard_normal(P[k].shape)).astype(np.float32)
    prompt = list(np.random.default_rng(12).integers(0, cfg.vocab_size, 7))
    toks, logits = U.CachedRunner(oracle, cfg, P, 32).generate(prompt, 4)
    ids = list(prompt)
    for t, lg in zip(toks, logits):
        ref = np_llama_logits(cfg, P, ids)[-1]
        assert rel(ref[None, :], np.asarray(lg).reshape(1, -1)) <= RTOL
        assert int(np.argmax(ref)) == t
        ids.append(t)


def test_llama_model_term_matches_numpy(oracle):
    """The reference-style term (no cache, argmax over every position, llama.rs:150-204)."""
    cfg = U.tiny_config(num_hidden_layers=2, tie_word_embeddings=False)
    P = U.param_arrays(cfg, seed=13, std=0.2)
    ids = np.random.default_rng(14).integers(0, cfg.vocab_size, (1, 9)).astype(np.uint32)
    it = U.interpreter(oracle, P)
    (y,) = it.run(U.llama.LlamaModel(cfg, 16).term(), [oracle.tensor(ids)])
    ref = np_llama_logits(cfg, P, list(ids[0]))
    srt = np.sort(ref, axis=-1)
    assert (srt[:, -1] - srt[:, -2]).min() > 1e-4 * np.abs(ref).max()  # no near tie in this sample
    assert np.array_equal(oracle.numpy(y).reshape(-1), np.argmax(ref, axis=-1))


def test_gemma_forward_matches_numpy(oracle):
    """Three layers: two local (window 5 of 9 tokens, local theta) and one global; batch 2."""
    cfg = MU.gemma_config()
    P = MU.gemma_params(cfg, seed=15, std=0.2)
    ids = np.random.default_rng(16).integers(0, cfg.vocab_size, (2, 9)).astype(np.uint32)
    it = U.interpreter(oracle, P)
    tok, logits = it.run(llm.gemma3.Gemma3Model(cfg, 9).term(), [oracle.tensor(ids)])
    ref = np_gemma_logits(cfg, P, ids)
    assert rel(ref, oracle.numpy(logits)) <= RTOL
    # each of the pieces this test is for moves the result by far more than the bar
    for tweak in ("window", "theta", "scale"):
        c2 = MU.gemma_config(**({"sliding_window": 0} if tweak == "window" else
                                {"rope_local_base_freq": cfg.rope_theta} if tweak == "theta" else {}))
        alt = np_gemma_logits(c2, P, ids) if tweak != "scale" else ref / np.sqrt(cfg.hidden_size)
        assert rel(alt, oracle.numpy(logits)) > 100 * RTOL, tweak

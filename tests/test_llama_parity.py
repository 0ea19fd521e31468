"""Llama end to end through the evaluator: reference-style full recompute vs the KV-cached
terms, and HIP vs the oracle (logits rel 1e-4 in f32 / 2e-2 in bf16, identical greedy tokens
over the first 32 steps in f32, with the top-1/top-2 margin recorded for tie-sensitive steps)."""
import numpy as np
import pytest

import llama_util as U
import parity
import vectors


def greedy_reference_style(be, cfg, arrays, prompt, steps):
    """catgrad-llm/examples/llama/main.rs:118-127: re-run the whole sequence per token."""
    it = U.interpreter(be, arrays)
    model = U.llama.LlamaModel(cfg, len(prompt) + steps)
    ids, toks = list(prompt), []
    for _ in range(steps):
        (y,) = it.run(model.term(), [be.tensor(np.asarray(ids, np.uint32).reshape(1, -1))])
        t = int(be.to_vec(y)[-1])
        toks.append(t)
        ids.append(t)
    return toks


def test_cached_equals_full_recompute_on_oracle(oracle):
    cfg = U.tiny_config()
    arrays = U.param_arrays(cfg, seed=1, std=0.2)
    prompt = list(np.random.default_rng(2).integers(0, cfg.vocab_size, 9))
    ref = greedy_reference_style(oracle, cfg, arrays, prompt, 6)
    got, _ = U.CachedRunner(oracle, cfg, arrays, 32).generate(prompt, 6)
    assert got == ref


def test_op_counts_of_emitters(oracle):
    """The emitted graph has the structure the reference emits: per-layer Backend-call count is
    constant and the model issues no op the trait lacks."""
    cfg1, cfg2 = U.tiny_config(num_hidden_layers=1), U.tiny_config(num_hidden_layers=2)
    a1, a2 = U.param_arrays(cfg1), U.param_arrays(cfg2)
    ids = oracle.tensor(np.zeros((1, 5), np.uint32))
    calls = []
    for cfg, arr in ((cfg1, a1), (cfg2, a2)):
        it = U.interpreter(oracle, arr)
        it.backend_calls()
        it.run(U.llama.LlamaModel(cfg, 16).term(), [ids])
        calls.append(it.backend_calls())
    per_layer = calls[1] - calls[0]
    assert 100 <= per_layer <= 160, per_layer      # ~130 Backend calls per Llama layer



@pytest.mark.gpu
def test_llama_f32_logits_and_tokens(oracle, hip):
    cfg = U.tiny_config(hidden_size=128, intermediate_size=256, num_hidden_layers=3, num_attention_heads=8,
                        num_key_value_heads=2, vocab_size=509)
    arrays = U.param_arrays(cfg, seed=3, std=0.1)
    prompt = list(np.random.default_rng(4).integers(0, cfg.vocab_size, 24))
    steps = 32
    rt, rl = U.CachedRunner(oracle, cfg, arrays, 64).generate(prompt, steps)
    gt, gl = U.CachedRunner(hip, cfg, arrays, 64).generate(prompt, steps)
    for i in range(steps):
        parity.assert_f32(rl[i], gl[i], f"step {i}")
        if rt[i] != gt[i]:
            # only acceptable when the oracle's own top-2 margin is inside the f32 error bound
            gap = parity.top2_gap_over_max(rl[i])[0]
            assert gap <= 2 * parity.RTOL_F32, f"step {i}: tokens differ, top-2 gap {gap}"
            break
    else:
        assert rt == gt


@pytest.mark.gpu
def test_llama_reference_style_on_hip(oracle, hip, hip_eager):
    cfg = U.tiny_config()
    arrays = U.param_arrays(cfg, seed=5, std=0.2)
    prompt = list(np.random.default_rng(6).integers(0, cfg.vocab_size, 11))
    ref = greedy_reference_style(oracle, cfg, arrays, prompt, 4)
    assert greedy_reference_style(hip, cfg, arrays, prompt, 4) == ref
    assert greedy_reference_style(hip_eager, cfg, arrays, prompt, 4) == ref
    got, _ = U.CachedRunner(hip, cfg, arrays, 32).generate(prompt, 4)
    assert got == ref


@pytest.mark.gpu
def test_llama_bf16_logits(oracle, hip_bf16):
    cfg = U.tiny_config(hidden_size=128, intermediate_size=256, num_hidden_layers=2, num_attention_heads=8,
                        num_key_value_heads=2, vocab_size=300)
    arrays = U.param_arrays(cfg, seed=7, std=0.1)
    # the oracle sees the same bf16-rounded parameters the device stores (rank >= 2 only)
    rounded = {}
    for k, a in arrays.items():
        if a.ndim >= 2:
            u = a.view(np.uint32).astype(np.uint64)
            a = (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)
        rounded[k] = a
    prompt = list(np.random.default_rng(8).integers(0, cfg.vocab_size, 40))
    r = U.CachedRunner(oracle, cfg, rounded, 64)
    g = U.CachedRunner(hip_bf16, cfg, arrays, 64)
    _, rl = r.prefill(prompt)
    _, gl = g.prefill(prompt)
    rl, gl = oracle.to_vec(rl), hip_bf16.to_vec(gl)
    parity.assert_bf16(rl, gl, "prefill")
    tok = int(np.argmax(rl))
    _, rl = r.step(tok)
    _, gl = g.step(tok)
    rl, gl = oracle.to_vec(rl), hip_bf16.to_vec(gl)
    parity.assert_bf16(rl, gl, "decode step")


@pytest.mark.gpu
def test_llama_prefill_of_many_rows(oracle, hip, hip_bf16):
    """A 256-token prompt: the sizes at which products are grouped, split along k with the residual
    added by the summing pass, gated activations applied by up_proj's GEMM, and blocks issued while
    the next is recorded.  f32 at 1e-4, bf16 at 2e-2, and the bf16 launch mix."""
    cfg = U.tiny_config(hidden_size=256, intermediate_size=512, num_hidden_layers=3, num_attention_heads=4,
                        num_key_value_heads=2, vocab_size=300)
    arrays = U.param_arrays(cfg, seed=11, std=0.05)
    rounded = {k: (vectors.bf16_round(a) if a.ndim >= 2 else a) for k, a in arrays.items()}
    prompt = list(np.random.default_rng(9).integers(0, cfg.vocab_size, 256))
    _, rl = U.CachedRunner(oracle, cfg, arrays, 300).prefill(prompt)
    _, gl = U.CachedRunner(hip, cfg, arrays, 300).prefill(prompt)
    rl, gl = oracle.to_vec(rl), hip.to_vec(gl)
    parity.assert_f32(rl, gl, "prefill of 256 rows")
    _, rl = U.CachedRunner(oracle, cfg, rounded, 300).prefill(prompt)
    g = U.CachedRunner(hip_bf16, cfg, arrays, 300)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    _, gl = g.prefill(prompt)
    rl, gl = oracle.to_vec(rl), hip_bf16.to_vec(gl)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    parity.assert_bf16(rl, gl, "prefill of 256 rows")
    launches = {k: v["launches"] for k, v in rep.items()}
    # per layer: q/k/v grouped, o_proj, gate_proj with up_proj (and the activation), down_proj = 4 GEMMs, and
    # the attention in one pass (in bf16 mode from 256 keys on)
    assert launches.get("gemm_mfma_bf16") == 4 * cfg.num_hidden_layers, launches
    assert launches.get("attn_prefill") == cfg.num_hidden_layers, launches
    assert "swiglu_fused" not in launches, launches


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,heads,kv_heads,layers", [(256, 8, 2, 2), (320, 4, 4, 2), (300, 4, 2, 2), (512, 16, 2, 2),
                                                         (1280, 16, 8, 1), (2048, 16, 16, 1), (2048, 32, 16, 1)])
def test_llama_prefill_rotates_in_the_projections_launch(oracle, hip_bf16, tokens, heads, kv_heads, layers):
    """bf16 prefill with heads of 64 (models/llama.rs:77-94, helpers.rs:195-221): the grouped q/k/v launch leaves the
    queries and keys rotated and a transposed bf16 copy of the values, so the trace holds neither a rotation nor a
    transposition of its own.  The caches it returns (rotated keys, values) and the logits of the prefill and of a
    decode step that reads those caches are held to the bf16 bar against the oracle on rounded parameters.  The
    sizes cover the tiles the launch may choose (128 x 64; 128 x 128 with eight waves, one or two workgroups to a
    CU, or with four waves) and a prompt that ends inside a tile."""
    cfg = U.tiny_config(hidden_size=64 * heads, intermediate_size=512, num_hidden_layers=layers,
                        num_attention_heads=heads, num_key_value_heads=kv_heads, vocab_size=300)
    arrays = U.param_arrays(cfg, seed=21, std=0.05)
    rounded = {k: (vectors.bf16_round(a) if a.ndim >= 2 else a) for k, a in arrays.items()}
    prompt = list(np.random.default_rng(tokens).integers(0, cfg.vocab_size, tokens))
    ref = U.CachedRunner(oracle, cfg, rounded, tokens + 8)
    rt, rl = ref.prefill(prompt)
    g = U.CachedRunner(hip_bf16, cfg, arrays, tokens + 8)
    hip_bf16.trace(2)
    hip_bf16.trace_reset()
    gt, gl = g.prefill(prompt)
    gl = hip_bf16.to_vec(gl)
    names = sorted(hip_bf16.trace_report())
    hip_bf16.trace(False)
    parity.assert_bf16(oracle.to_vec(rl), gl, "prefill logits")
    assert sum("grouped,rope" in n for n in names) >= 1, names
    # (300 keys are not a multiple of 8: that attention runs as two products and a softmax, which lay out the
    # values for themselves)
    assert not any(n.startswith(("rope_fused", "transpose_cast_bf16")) for n in names) or tokens % 8, names
    for layer in range(cfg.num_hidden_layers):
        for which, what in ((0, "rotated keys"), (1, "values")):
            parity.assert_bf16(oracle.to_vec(ref.kv[2 * layer + which]), hip_bf16.to_vec(g.kv[2 * layer + which]),
                               f"layer {layer} {what}")
    tok = int(oracle.to_vec(rt).reshape(-1)[0])
    _, rl = ref.step(tok)
    _, gl = g.step(tok)
    parity.assert_bf16(oracle.to_vec(rl), hip_bf16.to_vec(gl), "decode step on the prefill's caches")


@pytest.mark.gpu
def test_llama_prefill_block_ends_at_full_width(oracle, hip, hip_bf16):
    """Two layers at the 1B model's widths (hidden 2048, FFN 8192, 32 / 8 heads of 64) over a 128-token prompt:
    o_proj and down_proj are split along k here, every `residual + linear(x)` is issued as soon as it is recorded
    and left as the slices of its product, and the RMSNorm that reads it sums them.  Logits against the oracle at
    the stated bars in both modes, and the bf16 trace shows the norms taking the slices."""
    cfg = U.tiny_config(hidden_size=2048, intermediate_size=8192, num_hidden_layers=2, num_attention_heads=32,
                        num_key_value_heads=8, vocab_size=512)
    arrays = U.param_arrays(cfg, seed=3, std=0.02)
    rounded = {k: (vectors.bf16_round(a) if a.ndim >= 2 else a) for k, a in arrays.items()}
    prompt = list(np.random.default_rng(4).integers(0, cfg.vocab_size, 128))
    for be, params, check in ((hip, arrays, parity.assert_f32), (hip_bf16, rounded, parity.assert_bf16)):
        _, rl = U.CachedRunner(oracle, cfg, params, 160).prefill(prompt)
        g = U.CachedRunner(be, cfg, arrays, 160)
        be.trace(2)
        be.trace_reset()
        _, gl = g.prefill(prompt)
        gl = be.to_vec(gl)
        names = set(be.trace_report())
        be.trace(False)
        check(oracle.to_vec(rl), gl, "prefill of 128 rows at full width")
        if be is hip_bf16:
            assert any(n.startswith("rmsnorm_fused[") and "k-slices" in n for n in names), sorted(names)


@pytest.mark.gpu
def test_pipelined_decode_gives_the_same_tokens(hip, hip_bf16):
    """Token fed back on the device and read one step behind (cg_tensor_prefetch) == the loop that
    reads every token before the next step; also that a prefetched read returns the right data."""
    cfg = U.tiny_config(hidden_size=128, intermediate_size=256, num_hidden_layers=3, num_attention_heads=8,
                        num_key_value_heads=2, vocab_size=509)
    arrays = U.param_arrays(cfg, seed=5, std=0.1)
    prompt = list(np.random.default_rng(6).integers(0, cfg.vocab_size, 17))
    for be in (hip, hip_bf16):
        sync_tokens, _ = U.CachedRunner(be, cfg, arrays, 64).generate(prompt, 24)
        piped = U.CachedRunner(be, cfg, arrays, 64).generate_pipelined(prompt, 24)
        assert piped == sync_tokens
    x = np.arange(1000, dtype=np.float32)
    t = hip.add(hip.tensor(x), hip.tensor(x))
    hip.prefetch(t)
    later = hip.mul(t, t)                       # more work queued behind the copy
    assert np.array_equal(hip.to_vec(t), x + x)
    assert np.array_equal(hip.to_vec(later), (x + x) * (x + x))
    big = hip.add(hip.tensor(np.ones(5000, np.float32)), hip.tensor(np.ones(5000, np.float32)))
    hip.prefetch(big)                           # too large for the pinned slot: falls back to the plain read
    assert np.array_equal(hip.to_vec(big), np.full(5000, 2.0, np.float32))


@pytest.fixture(scope="module")
def llama_1b():
    """The north-star model at its real shape (16 layers, hidden 2048, 32/8 heads of 64, FFN 8192, vocabulary
    128256, tied lm_head) with the benchmark's parameters (seed 0, N(0, 0.02)) and a 16-token prompt."""
    llm = U.llm
    cfg = llm.random_init.llama_1b_config(llm.Config, 16)
    arrays = llm.random_init.llama_params(cfg, seed=0, std=0.02)
    prompt = [int(t) for t in np.random.default_rng(1).integers(0, cfg.vocab_size, 16)]
    return cfg, arrays, prompt


@pytest.mark.gpu
def test_llama_1b_full_shape_f32(oracle, hip, llama_1b):
    """f32 at the real shape: a 16-token prompt and 3 KV-cached decode steps, HIP against the oracle run here.
    Logits rel 1e-4, identical tokens; the oracle's top-1/top-2 gap is recorded so that a token flip on a
    near tie would be told apart from an error.  (About half a minute of oracle time.)"""
    cfg, arrays, prompt = llama_1b
    steps = 4                                         # the prefill's token + 3 decode steps
    rt, rl = U.CachedRunner(oracle, cfg, arrays, 32).generate(prompt, steps)
    gt, gl = U.CachedRunner(hip, cfg, arrays, 32).generate(prompt, steps)
    gaps = [float(parity.top2_gap_over_max(a)[0]) for a in rl]
    for i in range(steps):
        parity.assert_f32(rl[i], gl[i], f"position {i} (top-2 gap {gaps[i]:.2e})")
    for i in range(steps):
        assert rt[i] == gt[i] or gaps[i] <= 2 * parity.RTOL_F32, (i, rt, gt, gaps)
        if rt[i] != gt[i]:
            break


@pytest.mark.gpu
def test_llama_1b_first_32_greedy_tokens_f32(hip, llama_1b):
    """The north star's token criterion at the real shape: the first 32 greedy tokens in f32 are the oracle's
    (tests/golden/llama1b_f32_tokens.json, written by tests/golden/make_llama1b_tokens.py from the oracle
    alone - the loop of catgrad-llm/examples/llama/main.rs:114-169 with the KV-cached terms).  A token may
    differ only where the oracle's own gap between its two best logits is inside the f32 bar; after such a
    step the sequences are different inputs and the comparison ends.  The recorded logits (the eight largest
    and 64 fixed columns per step) are held to 1e-4 of max(|logit|, rms of the row)."""
    import json
    import os
    cfg, arrays, prompt = llama_1b
    g = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "llama1b_f32_tokens.json")))
    assert g["prompt"] == prompt
    steps = g["steps"]
    assert len(steps) == 32
    gt, gl = U.CachedRunner(hip, cfg, arrays, 64).generate(prompt, len(steps))
    for i, st in enumerate(steps):
        row = np.asarray(gl[i], np.float64).reshape(-1)
        cols = np.asarray(st["top8_cols"] + g["sample_cols"])
        ref = np.asarray(st["top8"] + st["sample"], np.float64)
        err = np.abs(row[cols] - ref) / np.maximum(np.abs(ref), st["rms"])
        assert err.max() <= parity.RTOL_F32, (i, float(err.max()))
        if gt[i] != st["token"]:
            assert st["gap_over_rms"] <= 2 * parity.RTOL_F32, (i, gt[i], st["token"], st["gap_over_rms"])
            break
    else:
        assert gt == [st["token"] for st in steps]


@pytest.mark.gpu
def test_llama_1b_full_shape_bf16(oracle, hip_bf16, llama_1b):
    """bf16 mode at the benchmarked shape: the prompt's logits and those of 3 KV-cached steps against the
    f32 oracle fed the parameters as the device stores them (rank >= 2 rounded to bf16), at the 2e-2 bar.
    Both sides are fed the oracle's tokens, so every position compares the same inputs."""
    cfg, arrays, prompt = llama_1b
    rounded = {k: (vectors.bf16_round(a) if a.ndim >= 2 else a) for k, a in arrays.items()}
    r = U.CachedRunner(oracle, cfg, rounded, 32)
    del rounded
    g = U.CachedRunner(hip_bf16, cfg, arrays, 32)
    tr, rl = r.prefill(prompt)
    _, gl = g.prefill(prompt)
    for i in range(4):
        rl, gl = oracle.to_vec(rl), hip_bf16.to_vec(gl)
        parity.assert_bf16(rl, gl, f"position {i}")
        tok = int(oracle.to_vec(tr)[0])
        if i < 3:
            tr, rl = r.step(tok)
            _, gl = g.step(tok)


@pytest.mark.gpu
def test_llama_steps_run_on_pattern_kernels(hip, hip_bf16):
    """No launch of a Llama prefill or decode step falls to the generic elementwise / row programs:
    every hot op is taken by a hand-written kernel (counted by kernel family, no tracing involved).
    A reordered emitter that made a matcher miss would show up here as "ew_fused" / "row_fused"."""
    cfg = U.tiny_config(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                        num_key_value_heads=2, vocab_size=512)
    arrays = U.param_arrays(cfg, seed=21, std=0.05)
    prompt = list(np.random.default_rng(22).integers(0, cfg.vocab_size, 48))
    layers = cfg.num_hidden_layers
    for be in (hip, hip_bf16):
        # a backend that has seen many sequence lengths before: the cache of aranges (which the sharing of the
        # per-layer masks builds on) must keep serving the lengths in use now
        for n in range(1000, 1040):
            assert be.to_vec(be.arange(n))[-1] == n - 1
        r = U.CachedRunner(be, cfg, arrays, 128)
        tok, _ = r.prefill(prompt)
        be.to_vec(tok)
        be.launch_counts(reset=True)
        tok, _ = r.prefill(prompt)
        be.to_vec(tok)
        pre = be.launch_counts(reset=True)
        assert not set(pre) & set(be.GENERIC_PROGRAMS), ("bf16" if be is hip_bf16 else "f32", sorted(pre.items()))
        assert pre.get("rmsnorm_fused") == 2 * layers + 1 and pre.get("rope_fused") == 2 * layers, pre
        tok, _ = r.step(int(be.to_vec(tok)[0]))
        be.to_vec(tok)
        be.launch_counts(reset=True)
        tok, _ = r.step(int(be.to_vec(tok)[0]))
        be.to_vec(tok)
        dec = be.launch_counts(reset=True)
        assert not set(dec) & set(be.GENERIC_PROGRAMS), dec
        gemv = "gemv_rowdot_bf16" if be is hip_bf16 else "gemv_rowdot_f32"
        # q/k/v, o_proj, gate + up, down_proj per layer and the lm_head; norms, RoPE, the gated activation,
        # residual adds and the cache append ride inside them and inside the attention launch
        products = dec.pop(gemv, 0) + dec.pop("gemm", 0)      # narrow products of this small shape take the tile kernel
        assert products == 4 * layers + 1, (products, dec)
        assert dec == {"attn_decode": layers, "gather": 1, "reduce_argmax": 1, "fill": 1}, dec

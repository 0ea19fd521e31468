"""Full-shape runs of BASELINE.json configs[3] (Qwen1.5-MoE-A2.7B layout) and configs[4] (Gemma-3-1B
shape) on one device, random init, bf16 weights.  No CPU oracle exists at these sizes (the
as-written MoE gathers 11.8 GB per projection on the CPU); what is checked here are properties that
do not depend on size: finite logits, tokens in range, and batch rows being independent (row r of a
batched run equals the same prompt run alone).  Parity against the oracle is at reduced shapes in
tests/test_moe_gemma_parity.py.
"""
import time

import numpy as np

import importlib

cg = importlib.import_module("catgrad-rs_amd")
_llm = importlib.import_module("catgrad-rs_amd.llm")
abi = cg.abi
Interpreter, Parameters, stdlib = cg.Interpreter, cg.Parameters, cg.stdlib
Config, gemma3, llama, qwen_moe = _llm.Config, _llm.gemma3, _llm.llama, _llm.qwen_moe


def _normal(g, shape, std, pool):
    """N(0, std) f32 of `shape`; big matrices come from a small pool of distinct draws (generating
    14 G normals on the host would take minutes and adds nothing to a throughput run)."""
    n = int(np.prod(shape))
    if n < (1 << 22):
        return g.standard_normal(shape, dtype=np.float32) * np.float32(std)
    slot = (tuple(shape), int(g.integers(0, 2)))
    if slot not in pool:
        pool[slot] = g.standard_normal(shape, dtype=np.float32) * np.float32(std)
    return pool[slot]


def qwen_moe_config(layers=24):
    return Config(hidden_size=2048, num_hidden_layers=layers, num_attention_heads=16, num_key_value_heads=16,
                  head_dim=128, vocab_size=151936, rms_norm_eps=1e-6, rope_theta=1000000.0, num_experts=60,
                  num_experts_per_tok=4, moe_intermediate_size=1408, shared_expert_intermediate_size=5632,
                  norm_topk_prob=False, tie_word_embeddings=False)


def qwen_moe_parameters(be, cfg, seed=0, std=0.02):
    g = np.random.default_rng(seed)
    pool = {}
    P = Parameters()
    h, e, f, sf, v = cfg.hidden_size, cfg.num_experts, cfg.moe_intermediate_size, \
        cfg.shared_expert_intermediate_size, cfg.vocab_size

    def w(name, shape, s=std):
        P[name] = be.tensor(_normal(g, shape, s, pool))
    w("qwen_moe.model.embed_tokens.weight", (v, h))
    w("qwen_moe.lm_head.weight", (v, h))
    P["qwen_moe.model.norm.weight"] = be.tensor(np.ones(h, np.float32))
    for i in range(cfg.num_hidden_layers):
        p = f"qwen_moe.model.layers.{i}."
        P[p + "input_layernorm.weight"] = be.tensor(np.ones(h, np.float32))
        P[p + "post_attention_layernorm.weight"] = be.tensor(np.ones(h, np.float32))
        for n in ("q_proj", "k_proj", "v_proj"):
            w(p + f"self_attn.{n}.weight", (h, h))
            w(p + f"self_attn.{n}.bias", (h,))
        w(p + "self_attn.o_proj.weight", (h, h))
        w(p + "mlp.gate.weight", (e, h))
        w(p + "mlp.experts.gate_proj.weight", (e, f, h))
        w(p + "mlp.experts.up_proj.weight", (e, f, h))
        w(p + "mlp.experts.down_proj.weight", (e, h, f))
        w(p + "mlp.shared_expert.gate_proj.weight", (sf, h))
        w(p + "mlp.shared_expert.up_proj.weight", (sf, h))
        w(p + "mlp.shared_expert.down_proj.weight", (h, sf))
        w(p + "mlp.shared_expert_gate.weight", (1, h))
    return P


def run_qwen_moe(lib, layers=24, batch=4, prompt=256, steps=64, warmup=2, count_experts=True):
    be = abi.Backend(lib, flags=abi.FLAG_BF16)
    cfg = qwen_moe_config(layers)
    t0 = time.time()
    P = qwen_moe_parameters(be, cfg)
    be.sync()
    setup_s = time.time() - t0
    r = _llm.CachedRunner(be, cfg, P, prompt + steps + warmup + 8, qwen_moe.QwenMoePrefill, qwen_moe.QwenMoeDecode)
    ids = np.random.default_rng(1).integers(0, cfg.vocab_size, (batch, prompt)).astype(np.uint32)
    # batch rows are independent: row 0 alone gives row 0 of the batch
    tok1, lg1 = r.prefill(ids[:1])
    alone = be.numpy(lg1)[0, 0]
    tok, lg = r.prefill(ids)                 # also the warm-up pass
    together = be.numpy(lg)
    assert np.all(np.isfinite(together)), "non-finite logits"
    rel = float(np.max(np.abs(together[0, 0] - alone)) / np.max(np.abs(alone)))
    assert rel <= 2e-2, f"row 0 of the batch differs from the prompt run alone: rel {rel}"
    be.sync()
    t = time.perf_counter()
    tok, lg = r.prefill(ids)
    be.to_vec(tok)
    prefill_s = time.perf_counter() - t
    toks = []
    for i in range(warmup + steps):
        if i == warmup:
            be.sync()
            launches0 = be.stats()["launches"]
            t = time.perf_counter()
        nxt, _ = r.step(tok)
        be.prefetch(nxt)
        toks.append(be.to_vec(tok).reshape(-1))
        tok = nxt
    toks.append(be.to_vec(tok).reshape(-1))
    be.sync()
    decode_s = time.perf_counter() - t
    launches = (be.stats()["launches"] - launches0) / steps
    toks = np.stack(toks)
    assert toks.max() < cfg.vocab_size
    # the experts a step really reads: a few more steps through a term that also returns its routing
    routed_term = qwen_moe.QwenMoeDecodeRouted(cfg).term()
    n_kv = 2 * cfg.num_hidden_layers
    distinct = []
    # (a kernel trace of the timed loop leaves these steps out: with the indices also returned, the expert
    # matrices are gathered as written)
    for _ in range(4 if count_experts else 0):
        out = r.it.run(routed_term, [be.reshape(tok, [batch, 1]), r.pos, r.cos, r.sin] + r.kv,
                       moved=range(4, 4 + n_kv))
        tok, r.kv, routing = out[0], out[2:2 + n_kv], out[2 + n_kv:]
        r.pos += 1
        distinct.append([len(np.unique(be.to_vec(ix))) for ix in routing])
    distinct_per_layer = float(np.mean(distinct)) if distinct else float(min(batch * cfg.num_experts_per_tok, cfg.num_experts))
    # bytes a decode step has to read: attention + shared expert + router + distinct routed experts
    h, f, sf, e = cfg.hidden_size, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size, cfg.num_experts
    if count_experts:
        del out, routing
    del r, P, tok, nxt, lg, lg1, tok1
    be.close()
    per_layer_fixed = (4 * h * h + 3 * sf * h + e * h) * 2
    expert_bytes = 3 * f * h * 2
    upper = layers * (per_layer_fixed + min(batch * cfg.num_experts_per_tok, e) * expert_bytes) + cfg.vocab_size * h * 2
    actual = layers * (per_layer_fixed + distinct_per_layer * expert_bytes) + cfg.vocab_size * h * 2
    return {"workload": "BASELINE configs[3]: Qwen1.5-MoE-A2.7B layout, random init N(0,0.02) (large matrices drawn "
                        f"from a pool of two per shape), bf16 weights, {layers} layers, batch {batch} x {prompt}-token "
                        f"prompts, {steps} greedy steps with KV cache",
            "decode_steps_per_s": steps / decode_s, "decode_tokens_per_s": steps * batch / decode_s,
            "ms_per_step": decode_s / steps * 1e3, "prefill_ms": prefill_s * 1e3,
            "prefill_tokens_per_s": batch * prompt / prefill_s, "kernel_launches_per_step": launches,
            "decode_weight_bytes_per_step_upper_bound": upper,
            "decode_hbm_fraction_at_upper_bound": upper * (steps / decode_s) / 8e12,
            "distinct_experts_per_layer_and_step": distinct_per_layer,
            "decode_weight_bytes_per_step": actual,
            "decode_hbm_fraction": actual * (steps / decode_s) / 8e12,
            "row_independence_rel_err": rel, "setup_s": setup_s}


def gemma3_config(layers=26):
    return Config(hidden_size=1152, intermediate_size=6912, num_hidden_layers=layers, num_attention_heads=4,
                  num_key_value_heads=1, head_dim=256, vocab_size=262144, rms_norm_eps=1e-6, rope_theta=1000000.0,
                  rope_local_base_freq=10000.0, sliding_window=512, sliding_window_pattern=6)


def gemma3_parameters(be, cfg, seed=0, std=0.02):
    g = np.random.default_rng(seed)
    pool = {}
    P = Parameters()
    h, hd, f = cfg.hidden_size, cfg.head_dim, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd

    def w(name, shape, s=std):
        P[name] = be.tensor(_normal(g, shape, s, pool))
    w("gemma3.model.embed_tokens.weight", (cfg.vocab_size, h))
    w("gemma3.model.norm.weight", (h,))
    for i in range(cfg.num_hidden_layers):
        p = f"gemma3.model.layers.{i}."
        for n in ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
                  "post_feedforward_layernorm"):
            w(p + n + ".weight", (h,))
        w(p + "self_attn.q_norm.weight", (hd,))
        w(p + "self_attn.k_norm.weight", (hd,))
        w(p + "self_attn.q_proj.weight", (q, h))
        w(p + "self_attn.k_proj.weight", (kv, h))
        w(p + "self_attn.v_proj.weight", (kv, h))
        w(p + "self_attn.o_proj.weight", (h, q))
        w(p + "mlp.gate_proj.weight", (f, h))
        w(p + "mlp.up_proj.weight", (f, h))
        w(p + "mlp.down_proj.weight", (h, f))
    return P


def run_gemma3(lib, layers=26, batch=8, prompt=2048, iters=3):
    be = abi.Backend(lib, flags=abi.FLAG_BF16)
    cfg = gemma3_config(layers)
    P = gemma3_parameters(be, cfg)
    it = Interpreter(be, stdlib(), P)
    term = gemma3.Gemma3Model(cfg, prompt, last_position_only=True).term()
    ids = np.random.default_rng(1).integers(0, cfg.vocab_size, (batch, prompt)).astype(np.uint32)
    dev_ids = be.tensor(ids)
    tok, lg = it.run(term, [dev_ids])
    together = be.numpy(lg)                                   # warm-up pass
    assert np.all(np.isfinite(together)), "non-finite logits"
    _, lg1 = it.run(term, [be.tensor(ids[3:4])])
    alone = be.numpy(lg1)[0, 0]
    rel = float(np.max(np.abs(together[3, 0] - alone)) / np.max(np.abs(alone)))
    assert rel <= 2e-2, f"row 3 of the batch differs from the prompt run alone: rel {rel}"
    be.sync()
    t = time.perf_counter()
    for _ in range(iters):
        tok, lg = it.run(term, [dev_ids])
        be.to_vec(tok)
    dt = (time.perf_counter() - t) / iters
    be.trace(True)
    be.trace_reset()
    tok, lg = it.run(term, [dev_ids])
    be.to_vec(tok)
    rep = be.trace_report()
    be.trace(False)
    total = sum(v["ms"] for v in rep.values()) or 1.0
    flops = sum(v["flops"] for v in rep.values())
    share = {k: round(v["ms"] / total, 4) for k, v in sorted(rep.items(), key=lambda kv: -kv[1]["ms"])[:8]}
    gm = rep.get("gemm_mfma_bf16")
    del it, P, tok, lg, lg1, dev_ids
    be.close()
    return {"workload": f"BASELINE configs[4]: Gemma-3-1B shape, random init N(0,0.02), bf16 weights, {layers} layers, "
                        f"batch {batch} x {prompt}-token prompts, prefill only, logits of the last position, 5 local "
                        "(window 512) : 1 global layers",
            "prefill_ms": dt * 1e3, "prefill_tokens_per_s": batch * prompt / dt, "matmul_flops": flops,
            "matmul_tflops_end_to_end": flops / dt / 1e12, "kernel_ms": total,
            "gemm_tflops": (gm["flops"] / (gm["ms"] * 1e-3) / 1e12) if gm else None,
            "kernel_time_share": share, "row_independence_rel_err": rel}

"""Seeded random-init parameters for the Qwen-MoE-layout and Gemma-3 modules."""
import importlib

import numpy as np

llm = importlib.import_module("catgrad-rs_amd.llm")


def qwen_moe_config(**kw):
    c = dict(hidden_size=64, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=4, head_dim=16,
             vocab_size=97, rms_norm_eps=1e-6, rope_theta=1000000.0, num_experts=8, num_experts_per_tok=2,
             moe_intermediate_size=48, shared_expert_intermediate_size=96, norm_topk_prob=False,
             tie_word_embeddings=False)
    c.update(kw)
    return llm.Config(**c)


def qwen_moe_params(cfg, seed=0, std=0.02):
    g = np.random.default_rng(seed)
    h, hd = cfg.hidden_size, cfg.get_head_dim()
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd
    e, f, sf = cfg.num_experts, cfg.moe_intermediate_size, cfg.shared_expert_intermediate_size
    out = {}

    def w(name, shape, s=std):
        out[name] = g.standard_normal(shape, dtype=np.float32) * np.float32(s)
    w("qwen_moe.model.embed_tokens.weight", (cfg.vocab_size, h))
    w("qwen_moe.lm_head.weight", (cfg.vocab_size, h))
    out["qwen_moe.model.norm.weight"] = np.ones(h, np.float32)
    for i in range(cfg.num_hidden_layers):
        p = f"qwen_moe.model.layers.{i}."
        out[p + "input_layernorm.weight"] = np.ones(h, np.float32)
        out[p + "post_attention_layernorm.weight"] = np.ones(h, np.float32)
        for n, o in (("q_proj", q), ("k_proj", kv), ("v_proj", kv)):
            w(p + f"self_attn.{n}.weight", (o, h))
            w(p + f"self_attn.{n}.bias", (o,))
        w(p + "self_attn.o_proj.weight", (h, q))
        w(p + "mlp.gate.weight", (e, h), 1.0)                 # spread the router logits
        w(p + "mlp.experts.gate_proj.weight", (e, f, h))
        w(p + "mlp.experts.up_proj.weight", (e, f, h))
        w(p + "mlp.experts.down_proj.weight", (e, h, f))
        w(p + "mlp.shared_expert.gate_proj.weight", (sf, h))
        w(p + "mlp.shared_expert.up_proj.weight", (sf, h))
        w(p + "mlp.shared_expert.down_proj.weight", (h, sf))
        w(p + "mlp.shared_expert_gate.weight", (1, h))
    return out


def gemma_config(**kw):
    c = dict(hidden_size=48, intermediate_size=96, num_hidden_layers=3, num_attention_heads=4,
             num_key_value_heads=1, head_dim=16, vocab_size=131, rms_norm_eps=1e-6, rope_theta=1000000.0,
             rope_local_base_freq=10000.0, sliding_window=5, sliding_window_pattern=3)
    c.update(kw)
    return llm.Config(**c)


def gemma_params(cfg, seed=0, std=0.02):
    g = np.random.default_rng(seed)
    h, hd, f = cfg.hidden_size, cfg.head_dim, cfg.intermediate_size
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd
    out = {}

    def w(name, shape, s=std):
        out[name] = g.standard_normal(shape, dtype=np.float32) * np.float32(s)
    w("gemma3.model.embed_tokens.weight", (cfg.vocab_size, h))
    w("gemma3.model.norm.weight", (h,), 0.1)
    for i in range(cfg.num_hidden_layers):
        p = f"gemma3.model.layers.{i}."
        for n in ("input_layernorm", "post_attention_layernorm", "pre_feedforward_layernorm",
                  "post_feedforward_layernorm"):
            w(p + n + ".weight", (h,), 0.1)
        w(p + "self_attn.q_norm.weight", (hd,), 0.1)
        w(p + "self_attn.k_norm.weight", (hd,), 0.1)
        w(p + "self_attn.q_proj.weight", (q, h))
        w(p + "self_attn.k_proj.weight", (kv, h))
        w(p + "self_attn.v_proj.weight", (kv, h))
        w(p + "self_attn.o_proj.weight", (h, q))
        w(p + "mlp.gate_proj.weight", (f, h))
        w(p + "mlp.up_proj.weight", (f, h))
        w(p + "mlp.down_proj.weight", (h, f))
    return out

"""Seeded random-init parameters of the Llama layout (BASELINE config 3: weights ~ N(0, std), norms = 1),
as numpy arrays by parameter path.  There are no checkpoints offline; benchmarks and tests draw from here."""
import numpy as np


def llama_params(cfg, seed=0, std=0.02):
    g = np.random.default_rng(seed)
    h, f, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    kv = h // (cfg.num_attention_heads // cfg.num_key_value_heads)
    out = {}

    def w(name, shape):
        out[name] = (g.standard_normal(shape, dtype=np.float32) * np.float32(std))

    def ones(name, n):
        out[name] = np.ones(n, np.float32)
    w("llama.model.embed_tokens.weight", (v, h))
    for i in range(cfg.num_hidden_layers):
        p = f"llama.model.layers.{i}."
        ones(p + "input_layernorm.weight", h)
        ones(p + "post_attention_layernorm.weight", h)
        w(p + "self_attn.q_proj.weight", (h, h))
        w(p + "self_attn.k_proj.weight", (kv, h))
        w(p + "self_attn.v_proj.weight", (kv, h))
        w(p + "self_attn.o_proj.weight", (h, h))
        w(p + "mlp.gate_proj.weight", (f, h))
        w(p + "mlp.up_proj.weight", (f, h))
        w(p + "mlp.down_proj.weight", (h, f))
    ones("llama.model.norm.weight", h)
    if not cfg.tie_word_embeddings:
        w("llama.lm_head.weight", (v, h))
    return out


def llama_1b_config(Config, layers=16):
    """The Llama-3.2-1B shape of BASELINE config 3."""
    return Config(hidden_size=2048, intermediate_size=8192, num_hidden_layers=layers,
                  num_attention_heads=32, num_key_value_heads=8, vocab_size=128256,
                  rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True)


def bf16_round(a):
    """f32 array rounded to the nearest bf16 (ties to even), as f32: what bf16 storage keeps."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)

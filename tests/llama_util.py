"""Shared helpers for the Llama parity tests: seeded random-init parameters and drivers."""
import importlib

import numpy as np

cg = importlib.import_module("catgrad-rs_amd")
llm = importlib.import_module("catgrad-rs_amd.llm")
llama = llm.llama


def tiny_config(**kw):
    c = dict(hidden_size=64, intermediate_size=160, num_hidden_layers=2, num_attention_heads=4,
             num_key_value_heads=2, vocab_size=211, rms_norm_eps=1e-5, rope_theta=500000.0,
             tie_word_embeddings=True)
    c.update(kw)
    return llm.Config(**c)


def param_arrays(cfg, seed=0, std=0.02):
    """weights ~ N(0, std), norms = 1 (BASELINE config 3), as numpy arrays by parameter path."""
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


def interpreter(be, arrays):
    P = cg.Parameters()
    for k, a in arrays.items():
        P[k] = be.tensor(a)
    return cg.Interpreter(be, cg.stdlib(), P)


class CachedRunner:
    """Greedy decoding with the KV-cached terms (prefill once, then one token per run)."""

    def __init__(self, be, cfg, arrays, max_positions, prefill_cls=None, decode_cls=None):
        """prefill_cls / decode_cls: the KV-cached term classes (default Llama's; the Qwen-MoE-layout
        ones take ids of shape [B, S])."""
        self.be, self.cfg = be, cfg
        self.prefill_cls = prefill_cls or llama.LlamaPrefill
        self.it = interpreter(be, arrays)
        self.cos, self.sin = self.it.run(llama.RopeTables(cfg).term(), [max_positions])
        self.decode_term = (decode_cls or llama.LlamaDecode)(cfg).term()
        self.kv = None
        self.pos = 0
        self._prefill_terms = {}

    def prefill(self, ids):
        ids = np.asarray(ids, np.uint32)
        ids = ids.reshape(1, -1) if ids.ndim == 1 else ids
        n = ids.shape[1]
        self.batch = ids.shape[0]
        if n not in self._prefill_terms:      # the term depends on the prompt length only
            self._prefill_terms[n] = self.prefill_cls(self.cfg, n).term()
        term = self._prefill_terms[n]
        out = self.it.run(term, [self.be.tensor(ids), self.cos, self.sin])
        self.kv = out[2:]
        self.pos = ids.shape[1]
        return out[0], out[1]

    def step(self, token):
        """`token`: an int, or the [1, 1, 1] token tensor of the previous step (stays on the device)."""
        if isinstance(token, cg.Tensor):
            ids = self.be.reshape(token, [self.batch, 1])
        else:
            ids = self.be.tensor(np.asarray(token, np.uint32).reshape(self.batch, 1))
        # the cache tensors are given away (Interpreter::run takes its values by value): the step may
        # then append to them in place
        out = self.it.run(self.decode_term, [ids, self.pos, self.cos, self.sin] + self.kv,
                          moved=range(4, 4 + len(self.kv)))
        self.kv = out[2:]
        self.pos += 1
        return out[0], out[1]

    def generate_pipelined(self, prompt, steps):
        """Greedy tokens with the sampled token fed back on the device and read one step behind:
        the host records and issues step t+1 while the device still runs step t."""
        tok, _ = self.prefill(prompt)
        self.be.prefetch(tok)
        toks, prev = [], tok
        for _ in range(steps - 1):
            tok, _ = self.step(prev)
            self.be.prefetch(tok)
            toks.append(int(self.be.to_vec(prev)[0]))
            prev = tok
        toks.append(int(self.be.to_vec(prev)[0]))
        return toks

    def generate(self, prompt, steps):
        """Returns (tokens, logits per step as numpy)."""
        tok, logits = self.prefill(prompt)
        toks, lg = [], []
        for _ in range(steps):
            t = int(self.be.to_vec(tok)[0])
            toks.append(t)
            lg.append(self.be.to_vec(logits))
            tok, logits = self.step(t)
        return toks, lg

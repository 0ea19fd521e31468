"""Llama as a catgrad `Module`.

`LlamaModel` mirrors catgrad-llm/src/models/llama.rs line for line: no KV cache, every step
re-runs the whole sequence, RoPE tables are rebuilt inside the graph, argmax over all positions.

`LlamaPrefill` / `LlamaDecode` are the KV-cached form of the same layer, written with the same
helpers in the order the legacy stack uses (catgrad-llm/src/legacy/models/llama.rs:63-128 and
legacy/models/utils.rs:210-228): RoPE on the un-repeated k, `concat(2, cached, new)`, repeat_kv,
last-position lm_head (legacy/models/llama.rs:38-42).  Cache tensors and RoPE tables are extra
term inputs/outputs; `pos` is a Nat input, so one term serves every decode step.
"""
import numpy as np

from ..lang import (Module, NAT, TENSOR, argmax, broadcast, concat, constant, matmul, make_shape,
                    path, reshape, shape, slice, transpose, unpack)
from ..nn import linear_b, silu, softmax
from .helpers import (Cache, apply_rope_embedding, causal_mask, embeddings, repeat_kv, rmsnorm,
                      rope_tables)


class LlamaModel(Module):
    def __init__(self, config, max_sequence_length):
        self.config = config
        self.max_sequence_length = max_sequence_length

    def path(self):
        return path(["llama"])

    def sort(self):
        return [TENSOR], [TENSOR]

    # Two seams for the decoders built on this layer (qwen_moe.py): how a linear is applied (the
    # reference's is batch-1, stdlib/nn/mod.rs:182-192) and how ids become the first activations.
    qkv_bias = False

    def linear(self, builder, in_dim, out_dim, p, x, bias=False):
        return linear_b(builder, in_dim, out_dim, bias, p, x)

    def embed(self, builder, ids):
        return embeddings(builder, self.path().extend(["model", "embed_tokens"]), ids)

    # models/llama.rs:11-35
    def mlp(self, builder, p, x):
        c = self.config
        gate = self.linear(builder, c.hidden_size, c.intermediate_size, p.extend(["gate_proj"]), x)
        up = self.linear(builder, c.hidden_size, c.intermediate_size, p.extend(["up_proj"]), x)
        x = silu(builder, gate) * up
        return self.linear(builder, c.intermediate_size, c.hidden_size, p.extend(["down_proj"]), x)

    def qkv(self, builder, p, x):
        c = self.config
        dim = c.hidden_size
        num_heads, num_kv_heads = c.num_attention_heads, c.num_key_value_heads
        head_dim = c.hidden_size // num_heads
        rep = num_heads // num_kv_heads
        b, s, _ = unpack(builder, 3, shape(builder, x))
        q = self.linear(builder, dim, dim, p.extend(["q_proj"]), x, bias=self.qkv_bias)
        k = self.linear(builder, dim, dim // rep, p.extend(["k_proj"]), x, bias=self.qkv_bias)
        v = self.linear(builder, dim, dim // rep, p.extend(["v_proj"]), x, bias=self.qkv_bias)
        sh = make_shape(builder, b, s, num_kv_heads, head_dim)
        k = reshape(builder, sh, k)
        v = reshape(builder, sh, v)
        sh = make_shape(builder, b, s, num_heads, head_dim)
        q = reshape(builder, sh, q)
        q = transpose(builder, 1, 2, q)
        k = transpose(builder, 1, 2, k)
        v = transpose(builder, 1, 2, v)
        return b, s, q, k, v

    def scores(self, builder, b, s, q, k, v, p):
        """models/llama.rs:95-112: scaled masked softmax attention and o_proj."""
        c = self.config
        dim = c.hidden_size
        head_dim = c.hidden_size // c.num_attention_heads
        tk = transpose(builder, 2, 3, k)
        attn = matmul(builder, q, tk)
        sh = shape(builder, attn)
        denom = constant(builder, float(np.sqrt(np.float32(head_dim))), sh)
        attn = attn / denom
        mask = causal_mask(builder, s)
        mask = broadcast(builder, mask, sh)
        attn = attn + mask
        attn = softmax(builder, attn)
        attn = matmul(builder, attn, v)
        attn = transpose(builder, 1, 2, attn)
        attn = reshape(builder, make_shape(builder, b, s, dim), attn)
        return self.linear(builder, dim, dim, p.extend(["o_proj"]), attn)

    # models/llama.rs:37-112
    def attention(self, builder, layer_id, cache, pos, p, x):
        c = self.config
        head_dim = c.hidden_size // c.num_attention_heads
        rep = c.num_attention_heads // c.num_key_value_heads
        b, s, q, k, v = self.qkv(builder, p, x)
        k = repeat_kv(builder, rep, k)
        v = repeat_kv(builder, rep, v)
        q = apply_rope_embedding(builder, pos, head_dim, cache.cos, cache.sin, q)
        k = apply_rope_embedding(builder, pos, head_dim, cache.cos, cache.sin, k)
        return self.scores(builder, b, s, q, k, v, p)

    # models/llama.rs:114-147
    def layer(self, builder, layer_id, cache, pos, p, x, attention=None):
        c = self.config
        res = x
        x = rmsnorm(builder, c.rms_norm_eps, p.extend(["input_layernorm"]), x)
        x = (attention or self.attention)(builder, layer_id, cache, pos, p.extend(["self_attn"]), x)
        x = res + x
        res = x
        x = rmsnorm(builder, c.rms_norm_eps, p.extend(["post_attention_layernorm"]), x)
        x = self.mlp(builder, p.extend(["mlp"]), x)
        return x + res

    def lm_head(self, builder, x):
        c = self.config
        root = self.path()
        w = ["model", "embed_tokens"] if c.tie_word_embeddings else ["lm_head"]
        return self.linear(builder, c.hidden_size, c.vocab_size, root.extend(w), x)

    # models/llama.rs:150-204
    def def_(self, builder, args):
        (x,) = args
        c = self.config
        root = self.path()
        cache = Cache.init(builder, c, self.max_sequence_length)
        x = self.embed(builder, x)
        for i in range(c.num_hidden_layers):
            x = self.layer(builder, i, cache, 0, root.extend(["model", "layers", i]), x)
        x = rmsnorm(builder, c.rms_norm_eps, root.extend(["model", "norm"]), x)
        x = self.lm_head(builder, x)
        x = argmax(builder, x)
        return [x]


class RopeTables(Module):
    """rope_tables as a term of its own (`usually precomputed`, helpers.rs:163): Nat -> cos, sin."""

    def __init__(self, config):
        self.config = config

    def path(self):
        return path(["rope_tables"])

    def sort(self):
        return [NAT], [TENSOR, TENSOR]

    def def_(self, builder, args):
        (n,) = args
        c = self.config
        return list(rope_tables(builder, c.rope_theta, n, c.get_head_dim()))


class _LlamaCached(LlamaModel):
    """Shared body of the KV-cached terms.  kv_in is None (prefill) or [(k, v)] per layer."""

    def run_layers(self, builder, ids, pos, cos, sin, kv_in):
        c = self.config
        root = self.path()
        cache = Cache(cos, sin)
        head_dim = c.hidden_size // c.num_attention_heads
        rep = c.num_attention_heads // c.num_key_value_heads
        kv_out = []

        def attention(builder, layer_id, cache, pos, p, x):
            b, s, q, k, v = self.qkv(builder, p, x)
            # legacy/models/llama.rs:103-110: rope, then cache update, then repeat_kv
            q = apply_rope_embedding(builder, pos, head_dim, cache.cos, cache.sin, q)
            k = apply_rope_embedding(builder, pos, head_dim, cache.cos, cache.sin, k)
            if kv_in is not None:
                ck, cv = kv_in[layer_id]
                k = concat(builder, 2, ck, k)          # legacy/models/utils.rs:222-223
                v = concat(builder, 2, cv, v)
            kv_out.append((k, v))
            kr = repeat_kv(builder, rep, k)
            vr = repeat_kv(builder, rep, v)
            return self.scores(builder, b, s, q, kr, vr, p)

        x = self.embed(builder, ids)
        for i in range(c.num_hidden_layers):
            x = self.layer(builder, i, cache, pos, root.extend(["model", "layers", i]), x,
                           attention=attention)
        x = rmsnorm(builder, c.rms_norm_eps, root.extend(["model", "norm"]), x)
        # logits for the last position only (legacy/models/llama.rs:38-42)
        _, s, _ = unpack(builder, 3, shape(builder, x))
        if kv_in is None:
            x = self.last_position(builder, x)
        x = self.lm_head(builder, x)
        tok = argmax(builder, x)
        flat = [t for kv in kv_out for t in kv]
        return tok, x, flat

    def last_position(self, builder, x):
        from ..lang import OP_NAT_ADD  # noqa: F401
        # narrow(1, tokens - 1, 1): the prompt length is static when the term is built
        return slice(builder, 1, self.prompt_len - 1, 1, x)


class LlamaPrefill(_LlamaCached):
    """ids[1,S], cos, sin -> token[1,1,1], logits[1,1,V], k0, v0, k1, v1, ..."""

    def __init__(self, config, prompt_len):
        super().__init__(config, prompt_len)
        self.prompt_len = prompt_len

    def sort(self):
        n = self.config.num_hidden_layers
        return [TENSOR, TENSOR, TENSOR], [TENSOR] * (2 + 2 * n)

    def def_(self, builder, args):
        ids, cos, sin = args
        tok, logits, kv = self.run_layers(builder, ids, 0, cos, sin, None)
        return [tok, logits] + kv


class LlamaDecode(_LlamaCached):
    """ids[1,1], pos: Nat, cos, sin, k0, v0, ... -> token, logits, k0', v0', ...
    The mask of a one-token step is causal_mask(1) = [[0]] broadcast over the cache length, as
    in the legacy stack (legacy/models/llama.rs:118-120)."""

    def __init__(self, config):
        super().__init__(config, 0)

    def sort(self):
        n = self.config.num_hidden_layers
        return [TENSOR, NAT, TENSOR, TENSOR] + [TENSOR] * (2 * n), [TENSOR] * (2 + 2 * n)

    def def_(self, builder, args):
        ids, pos, cos, sin = args[:4]
        kv = args[4:]
        kv_in = [(kv[2 * i], kv[2 * i + 1]) for i in range(self.config.num_hidden_layers)]
        tok, logits, kv_out = self.run_layers(builder, ids, pos, cos, sin, kv_in)
        return [tok, logits] + kv_out

"""A Qwen1.5-MoE-layout decoder as a catgrad `Module` (BASELINE config 4).

The reference has no model with this exact layout: its Qwen3-MoE has no shared expert
(catgrad-llm/src/models/qwen3.rs:64-133) and DeepSeek's shared expert has no gate
(catgrad-llm/src/models/deepseek.rs:163-165).  This module is build-authored from those pieces:
the routed experts are qwen3.rs's `moe` emitted op for op (router linear -> softmax -> topk ->
per-slot index of the stacked expert matrices -> matmul -> SwiGLU -> weighted sum), the shared
expert is deepseek's `mlp(shared_experts)` multiplied by `sigmoid(linear(H -> 1))`, attention is
llama's.  The reference models are batch-1 only (stdlib/nn/mod.rs:182-192 reshapes the weight to
[batch, in, out]); batches are handled here by folding [B, S, H] to [1, B*S, H] around every
linear and the MoE block, which uses only the reference's ops and is exact (tokens are
independent there).
"""
import numpy as np

from ..lang import (Module, TENSOR, argmax, broadcast, constant, get, index, make_shape, matmul,
                    param, path, reshape, shape, sum, topk, transpose, unpack)
from ..nn import linear_b, linear_no_bias, sigmoid, silu, softmax
from .helpers import (Cache, apply_rope_embedding, causal_mask, embeddings, repeat_kv, rmsnorm,
                      unsqueeze)


def fold_batch(builder, x):
    """[B, S, H] -> ([1, B*S, H], B, S)"""
    b, s, h = unpack(builder, 3, shape(builder, x))
    return reshape(builder, make_shape(builder, 1, b * s, h), x), b, s


def unfold_batch(builder, b, s, x):
    _, _, h = unpack(builder, 3, shape(builder, x))
    return reshape(builder, make_shape(builder, b, s, h), x)


class QwenMoeParts:
    """The pieces shared by the full-recompute model below and the KV-cached terms: batch-folding
    linear, routed experts + gated shared expert."""

    def linear(self, builder, i, o, p, x, bias=False):
        f, b, s = fold_batch(builder, x)
        y = linear_b(builder, i, o, bias, p, f)
        return unfold_batch(builder, b, s, y)

    def dense_mlp(self, builder, ffn, p, x):
        c = self.config
        gate = linear_no_bias(builder, c.hidden_size, ffn, p.extend(["gate_proj"]), x)
        up = linear_no_bias(builder, c.hidden_size, ffn, p.extend(["up_proj"]), x)
        x = silu(builder, gate) * up
        return linear_no_bias(builder, ffn, c.hidden_size, p.extend(["down_proj"]), x)

    # qwen3.rs:64-133, on x of shape [1, tokens, H]
    def moe(self, builder, p, x):
        c = self.config
        _, seq_len, _ = unpack(builder, 3, shape(builder, x))
        gate_all = param(builder, p.extend(["experts", "gate_proj", "weight"]))
        up_all = param(builder, p.extend(["experts", "up_proj", "weight"]))
        down_all = param(builder, p.extend(["experts", "down_proj", "weight"]))
        routed = linear_no_bias(builder, c.hidden_size, c.num_experts, p.extend(["gate"]), x)
        routed = softmax(builder, routed)
        values, indices = topk(builder, c.num_experts_per_tok, routed)
        sh = make_shape(builder, seq_len, c.num_experts_per_tok)
        indices = reshape(builder, sh, indices)
        values = reshape(builder, sh, values)
        if getattr(self, "routing_out", None) is not None:   # (a term that also returns its routing, below)
            self.routing_out.append(indices)
        if c.norm_topk_prob:
            sv = broadcast(builder, sum(builder, values), sh)
            values = values / sv
        fullx = transpose(builder, 0, 1, x)
        sumk = constant(builder, 0.0, shape(builder, fullx))
        for i in range(c.num_experts_per_tok):
            idx = get(builder, 1, i, indices)
            val = get(builder, 1, i, values)
            gate = index(builder, 0, idx, gate_all)
            up = index(builder, 0, idx, up_all)
            down = index(builder, 0, idx, down_all)
            gate = transpose(builder, 1, 2, gate)
            up = transpose(builder, 1, 2, up)
            down = transpose(builder, 1, 2, down)
            g = matmul(builder, fullx, gate)
            u = matmul(builder, fullx, up)
            h = silu(builder, g) * u
            h = matmul(builder, h, down)
            v = unsqueeze(builder, 2, 2, val)
            v = broadcast(builder, v, shape(builder, h))
            sumk = sumk + h * v
        sumk = transpose(builder, 0, 1, sumk)
        # shared expert (deepseek.rs:163-165) with Qwen1.5-MoE's sigmoid gate
        shared = self.dense_mlp(builder, c.shared_expert_intermediate_size, p.extend(["shared_expert"]), x)
        sg = linear_no_bias(builder, c.hidden_size, 1, p.extend(["shared_expert_gate"]), x)
        sg = broadcast(builder, sigmoid(builder, sg), shape(builder, shared))
        return sumk + shared * sg



class QwenMoeModel(QwenMoeParts, Module):
    def __init__(self, config, max_sequence_length, last_position_only=False):
        self.config = config
        self.max_sequence_length = max_sequence_length
        self.last_position_only = last_position_only

    def path(self):
        return path(["qwen_moe"])

    def sort(self):
        return [TENSOR], [TENSOR, TENSOR]

    def attention(self, builder, cache, pos, p, x):
        c = self.config
        dim, heads, kvh, hd = c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.get_head_dim()
        rep = heads // kvh
        b, s, _ = unpack(builder, 3, shape(builder, x))
        q = self.linear(builder, dim, heads * hd, p.extend(["q_proj"]), x, bias=True)
        k = self.linear(builder, dim, kvh * hd, p.extend(["k_proj"]), x, bias=True)
        v = self.linear(builder, dim, kvh * hd, p.extend(["v_proj"]), x, bias=True)
        q = transpose(builder, 1, 2, reshape(builder, make_shape(builder, b, s, heads, hd), q))
        k = transpose(builder, 1, 2, reshape(builder, make_shape(builder, b, s, kvh, hd), k))
        v = transpose(builder, 1, 2, reshape(builder, make_shape(builder, b, s, kvh, hd), v))
        k = repeat_kv(builder, rep, k)
        v = repeat_kv(builder, rep, v)
        q = apply_rope_embedding(builder, pos, hd, cache.cos, cache.sin, q)
        k = apply_rope_embedding(builder, pos, hd, cache.cos, cache.sin, k)
        attn = matmul(builder, q, transpose(builder, 2, 3, k))
        sh = shape(builder, attn)
        attn = attn / constant(builder, float(np.sqrt(np.float32(hd))), sh)
        attn = attn + broadcast(builder, causal_mask(builder, s), sh)
        attn = matmul(builder, softmax(builder, attn), v)
        attn = reshape(builder, make_shape(builder, b, s, heads * hd), transpose(builder, 1, 2, attn))
        return self.linear(builder, heads * hd, dim, p.extend(["o_proj"]), attn)

    def layer(self, builder, cache, pos, p, x):
        c = self.config
        res = x
        x = rmsnorm(builder, c.rms_norm_eps, p.extend(["input_layernorm"]), x)
        x = res + self.attention(builder, cache, pos, p.extend(["self_attn"]), x)
        res = x
        x = rmsnorm(builder, c.rms_norm_eps, p.extend(["post_attention_layernorm"]), x)
        f, b, s = fold_batch(builder, x)
        x = unfold_batch(builder, b, s, self.moe(builder, p.extend(["mlp"]), f))
        return x + res

    def def_(self, builder, args):
        """ids [B, S] -> (argmax tokens, logits)"""
        (ids,) = args
        c = self.config
        root = self.path()
        cache = Cache.init(builder, c, self.max_sequence_length)
        b, s = unpack(builder, 2, shape(builder, ids))
        x = embeddings(builder, root.extend(["model", "embed_tokens"]), ids)   # [1, B*S, H]
        x = reshape(builder, make_shape(builder, b, s, c.hidden_size), x)
        for i in range(c.num_hidden_layers):
            x = self.layer(builder, cache, 0, root.extend(["model", "layers", i]), x)
        x = rmsnorm(builder, c.rms_norm_eps, root.extend(["model", "norm"]), x)
        if self.last_position_only:
            from ..lang import slice as slice_
            x = slice_(builder, 1, self.max_sequence_length - 1, 1, x)
        logits = self.linear(builder, c.hidden_size, c.vocab_size, root.extend(["lm_head"]), x)
        return [argmax(builder, logits), logits]


# ---- KV-cached terms (BASELINE config 4: batch 4 x 256-token prompts, 64 greedy steps) -----------------
# The same cached layer as llama.LlamaPrefill / LlamaDecode (rope, concat(2, cached, new), repeat_kv,
# last-position lm_head), with this model's linear (q/k/v bias, batch folded into the sequence
# axis) and the MoE block in place of the dense MLP.
from . import llama as _llama  # noqa: E402


class _QwenMoeCachedParts(QwenMoeParts):
    qkv_bias = True

    def path(self):
        return path(["qwen_moe"])

    def embed(self, builder, ids):
        b, s = unpack(builder, 2, shape(builder, ids))
        x = embeddings(builder, self.path().extend(["model", "embed_tokens"]), ids)
        return reshape(builder, make_shape(builder, b, s, self.config.hidden_size), x)

    def mlp(self, builder, p, x):
        f, b, s = fold_batch(builder, x)
        return unfold_batch(builder, b, s, self.moe(builder, p, f))


class QwenMoePrefill(_QwenMoeCachedParts, _llama.LlamaPrefill):
    """ids[B,S], cos, sin -> token[B,1,1], logits[B,1,V], k0, v0, ..."""


class QwenMoeDecode(_QwenMoeCachedParts, _llama.LlamaDecode):
    """ids[B,1], pos: Nat, cos, sin, k0, v0, ... -> token, logits, k0', v0', ..."""


class QwenMoeDecodeRouted(QwenMoeDecode):
    """QwenMoeDecode that also returns every layer's expert indices [B, k] after the caches (for counting
    the distinct experts a step reads; not the term the benchmarks time)."""

    def sort(self):
        i, o = super().sort()
        return i, o + [TENSOR] * self.config.num_hidden_layers

    def def_(self, builder, args):
        self.routing_out = []
        out = super().def_(builder, args)
        routing, self.routing_out = self.routing_out, None
        return out + routing

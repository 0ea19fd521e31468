"""Gemma-3 as a catgrad `Module` (BASELINE config 5).

Mirrors catgrad-llm/src/models/gemma3.rs (QK-RMSNorm with the (1 + gamma) form, GeGLU, four
norms per layer, embedding scaled by sqrt(hidden), per-layer RoPE base).  Two things the
reference lacks are build-authored from its own ops: batches > 1 (linears run on the batch folded
into the sequence axis, see qwen_moe.fold_batch) and the sliding-window mask of the local layers
(the reference uses the plain causal mask everywhere, gemma3.rs:153-174): `sliding_window > 0`
adds `lt(window - 1, row - col)` to the causal mask, built from arange/lt/cast like
helpers.causal_mask.
"""
import numpy as np

from .. import abi
from ..lang import (Module, TENSOR, arange, argmax, broadcast, cast, constant, lt, make_shape, matmul,
                    nat_to_u32, pack, param, path, reshape, shape, slice, sum, to_nat, transpose,
                    unpack, dtype)
from ..nn import gelu, linear_no_bias, softmax, sqrt
from .helpers import F32_MIN, causal_mask, embeddings, repeat_kv, rope
from .qwen_moe import fold_batch, unfold_batch


class Gemma3Model(Module):
    def __init__(self, config, max_sequence_length, last_position_only=False):
        self.config = config
        self.max_sequence_length = max_sequence_length
        self.last_position_only = last_position_only

    def path(self):
        return path(["gemma3"])

    def sort(self):
        return [TENSOR], [TENSOR, TENSOR]

    def linear(self, builder, i, o, p, x):
        f, b, s = fold_batch(builder, x)
        return unfold_batch(builder, b, s, linear_no_bias(builder, i, o, p, f))

    # gemma3.rs:41-58 (rank-generic)
    def rmsnorm_raw(self, builder, n_rank, eps, x):
        x_shape = shape(builder, x)
        n = unpack(builder, n_rank, x_shape)[n_rank - 1]
        s = sum(builder, x * x)
        constn = cast(builder, nat_to_u32(builder, n), dtype(builder, x))
        constn = broadcast(builder, constn, shape(builder, s))
        mean = s / constn
        epsilon = constant(builder, eps, shape(builder, mean))
        rms = sqrt(builder, mean + epsilon)
        return x / broadcast(builder, rms, x_shape)

    # gemma3.rs:60-68
    def rmsnorm(self, builder, n_rank, eps, p, x):
        gamma = param(builder, p.extend(["weight"]))
        lr = self.rmsnorm_raw(builder, n_rank, eps, x)
        gamma = broadcast(builder, gamma, shape(builder, lr))
        one = constant(builder, 1.0, shape(builder, gamma))
        return lr * (one + gamma)

    def mlp(self, builder, p, x):
        c = self.config
        gate = self.linear(builder, c.hidden_size, c.intermediate_size, p.extend(["gate_proj"]), x)
        up = self.linear(builder, c.hidden_size, c.intermediate_size, p.extend(["up_proj"]), x)
        x = gelu(builder, gate) * up
        return self.linear(builder, c.intermediate_size, c.hidden_size, p.extend(["down_proj"]), x)

    def window_mask(self, builder, size, window):
        """f32::MIN where col > row (causal) or row - col >= window; 0 elsewhere."""
        mask = causal_mask(builder, size)
        sh = pack(builder, [size, size])
        col = broadcast(builder, arange(builder, size), sh)
        row = arange(builder, size)
        row = reshape(builder, pack(builder, [size, to_nat(builder, 1)]), row)
        row = broadcast(builder, row, sh)
        # col + window <= row  <=>  col + (window - 1) < row   (u32, no underflow)
        w = broadcast(builder, nat_to_u32(builder, to_nat(builder, window - 1)), sh)
        far = cast(builder, lt(builder, col + w, row), abi.F32)
        return mask + far * constant(builder, F32_MIN, shape(builder, far))

    # gemma3.rs:70-196
    def attention(self, builder, layer_id, pos, p, x):
        c = self.config
        dim, heads, kvh, hd = c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim
        rep = heads // kvh
        b, s, _ = unpack(builder, 3, shape(builder, x))
        q = self.linear(builder, dim, heads * hd, p.extend(["q_proj"]), x)
        k = self.linear(builder, dim, kvh * hd, p.extend(["k_proj"]), x)
        v = self.linear(builder, dim, kvh * hd, p.extend(["v_proj"]), x)
        q = transpose(builder, 1, 2, reshape(builder, make_shape(builder, b, s, heads, hd), q))
        k = transpose(builder, 1, 2, reshape(builder, make_shape(builder, b, s, kvh, hd), k))
        v = transpose(builder, 1, 2, reshape(builder, make_shape(builder, b, s, kvh, hd), v))
        q = reshape(builder, make_shape(builder, b * s * to_nat(builder, heads), hd), q)
        k = reshape(builder, make_shape(builder, b * s * to_nat(builder, kvh), hd), k)
        q = self.rmsnorm(builder, 2, c.rms_norm_eps, p.extend(["q_norm"]), q)
        k = self.rmsnorm(builder, 2, c.rms_norm_eps, p.extend(["k_norm"]), k)
        q = reshape(builder, make_shape(builder, b, heads, s, hd), q)
        k = reshape(builder, make_shape(builder, b, kvh, s, hd), k)
        local = (layer_id + 1) % c.sliding_window_pattern != 0
        theta = c.rope_local_base_freq if local else c.rope_theta
        q = rope(builder, theta, pos, s, hd, q)
        k = rope(builder, theta, pos, s, hd, k)
        k = repeat_kv(builder, rep, k)
        v = repeat_kv(builder, rep, v)
        attn = matmul(builder, q, transpose(builder, 2, 3, k))
        sh = shape(builder, attn)
        attn = attn / constant(builder, float(np.sqrt(np.float32(hd))), sh)
        if local and c.sliding_window > 0:
            mask = self.window_mask(builder, s, c.sliding_window)
        else:
            mask = causal_mask(builder, s)
        attn = attn + broadcast(builder, mask, sh)
        attn = matmul(builder, softmax(builder, attn), v)
        attn = reshape(builder, make_shape(builder, b, s, heads * hd), transpose(builder, 1, 2, attn))
        return self.linear(builder, heads * hd, dim, p.extend(["o_proj"]), attn)

    # gemma3.rs:198-240
    def layer(self, builder, layer_id, pos, p, x):
        e = self.config.rms_norm_eps
        res = x
        x = self.rmsnorm(builder, 3, e, p.extend(["input_layernorm"]), x)
        x = self.attention(builder, layer_id, pos, p.extend(["self_attn"]), x)
        x = self.rmsnorm(builder, 3, e, p.extend(["post_attention_layernorm"]), x)
        x = res + x
        res = x
        x = self.rmsnorm(builder, 3, e, p.extend(["pre_feedforward_layernorm"]), x)
        x = self.mlp(builder, p.extend(["mlp"]), x)
        x = self.rmsnorm(builder, 3, e, p.extend(["post_feedforward_layernorm"]), x)
        return x + res

    # gemma3.rs:248-292
    def def_(self, builder, args):
        (ids,) = args
        c = self.config
        root = self.path()
        b, s = unpack(builder, 2, shape(builder, ids))
        x = embeddings(builder, root.extend(["model", "embed_tokens"]), ids)
        x = reshape(builder, make_shape(builder, b, s, c.hidden_size), x)
        x = x * constant(builder, float(np.sqrt(np.float32(c.hidden_size))), shape(builder, x))
        for i in range(c.num_hidden_layers):
            x = self.layer(builder, i, 0, root.extend(["model", "layers", i]), x)
        x = self.rmsnorm(builder, 3, c.rms_norm_eps, root.extend(["model", "norm"]), x)
        if self.last_position_only:   # legacy/models/llama.rs:38-42: logits of the last position only
            x = slice(builder, 1, self.max_sequence_length - 1, 1, x)
        logits = self.linear(builder, c.hidden_size, c.vocab_size, root.extend(["model", "embed_tokens"]), x)
        return [argmax(builder, logits), logits]

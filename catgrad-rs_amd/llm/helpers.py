"""Mirror of catgrad-llm/src/helpers.rs: the op sequences of rmsnorm, layernorm, RoPE, causal
mask, repeat_kv and embeddings, emitted exactly as the reference emits them."""
from dataclasses import dataclass

import numpy as np

from .. import abi
from ..lang import (arange, broadcast, cast, concat, constant, cos, index, inverse, lt, make_shape,
                    nat_to_u32, pack, param, pow, reshape, shape, sin, slice, sum, to_nat, unpack,
                    dtype)
from ..nn import sqrt

F32_MIN = float(np.finfo(np.float32).min)


@dataclass
class Config:
    """The fields of legacy::models::utils::Config (utils.rs:52-112) the Interpreter-path models
    read."""
    hidden_size: int = 0
    intermediate_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    vocab_size: int = 0
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    tie_word_embeddings: bool = True
    head_dim: int = 0
    # MoE (Qwen-MoE layout)
    num_experts: int = 0
    num_experts_per_tok: int = 0
    moe_intermediate_size: int = 0
    shared_expert_intermediate_size: int = 0
    norm_topk_prob: bool = False
    # Gemma-3
    sliding_window: int = 0
    sliding_window_pattern: int = 6
    rope_local_base_freq: float = 10000.0
    query_pre_attn_scalar: float = 0.0

    def get_head_dim(self):
        return self.head_dim if self.head_dim else self.hidden_size // self.num_attention_heads


class Cache:
    """helpers.rs:27-43: only the RoPE tables live here on the Interpreter path."""

    def __init__(self, cos, sin):
        self.cos, self.sin = cos, sin

    @staticmethod
    def init(builder, config, positions):
        c, s = rope_tables(builder, config.rope_theta, to_nat(builder, positions),
                           config.get_head_dim())
        return Cache(c, s)


# helpers.rs:45-67
def chunk(builder, dim, chunks, chunk_size, x):
    return [slice(builder, dim, i * chunk_size, chunk_size, x) for i in range(chunks)]


def split(builder, dim, sizes, x):
    out, offset = [], 0
    for size in sizes:
        out.append(slice(builder, dim, offset, size, x))
        offset += size
    return out


# helpers.rs:69-84
def squeeze(builder, n, dim, x):
    s = list(unpack(builder, n, shape(builder, x)))
    s.pop(dim)
    return reshape(builder, pack(builder, s), x)


def unsqueeze(builder, n, dim, x):
    s = list(unpack(builder, n, shape(builder, x)))
    s.insert(dim, to_nat(builder, 1))
    return reshape(builder, pack(builder, s), x)


# helpers.rs:86-105
def layernorm_raw(builder, eps, x):
    x_shape = shape(builder, x)
    _, _, n = unpack(builder, 3, x_shape)
    s = sum(builder, x)
    constn = nat_to_u32(builder, n)
    constn = cast(builder, constn, dtype(builder, x))
    sh = shape(builder, s)
    constn = broadcast(builder, constn, sh)
    mean = s / constn
    nom = x - broadcast(builder, mean, x_shape)
    var = sum(builder, nom * nom) / constn
    sh = shape(builder, var)
    epsilon = constant(builder, eps, sh)
    stddev = sqrt(builder, var + epsilon)
    denom = broadcast(builder, stddev, x_shape)
    return nom / denom


# helpers.rs:107-118
def layernorm(builder, eps, p, x):
    gamma = param(builder, p.extend(["weight"]))
    lr = layernorm_raw(builder, eps, x)
    lr_shape = shape(builder, lr)
    gamma = broadcast(builder, gamma, lr_shape)
    lr = lr * gamma
    beta = param(builder, p.extend(["bias"]))
    beta = broadcast(builder, beta, lr_shape)
    return lr + beta


# helpers.rs:120-136
def rmsnorm_raw(builder, eps, x):
    x_shape = shape(builder, x)
    _, _, n = unpack(builder, 3, x_shape)
    s = sum(builder, x * x)
    constn = nat_to_u32(builder, n)
    constn = cast(builder, constn, dtype(builder, x))
    sh = shape(builder, s)
    constn = broadcast(builder, constn, sh)
    mean = s / constn
    epsilon = constant(builder, eps, shape(builder, mean))
    rms = sqrt(builder, mean + epsilon)
    denom = broadcast(builder, rms, x_shape)
    return x / denom


# helpers.rs:138-145
def rmsnorm(builder, eps, p, x):
    gamma = param(builder, p.extend(["weight"]))
    lr = rmsnorm_raw(builder, eps, x)
    lr_shape = shape(builder, lr)
    gamma = broadcast(builder, gamma, lr_shape)
    return lr * gamma


# helpers.rs:147-161
def repeat_kv(builder, rep, x):
    b, num_kv_heads, s, head_dim = unpack(builder, 4, shape(builder, x))
    x = reshape(builder, make_shape(builder, b, num_kv_heads, 1, s, head_dim), x)
    x = broadcast(builder, x, make_shape(builder, b, num_kv_heads, rep, s, head_dim))
    rnkv = num_kv_heads * to_nat(builder, rep)
    return reshape(builder, make_shape(builder, b, rnkv, s, head_dim), x)


# helpers.rs:163-193
def rope_tables(builder, theta, seq_len, head_dim):
    half_dim = head_dim // 2
    f = arange(builder, half_dim)
    f = cast(builder, f, abi.F32)
    sh = shape(builder, f)
    two = constant(builder, float(np.float32(2.0) / np.float32(head_dim)), sh)
    f = f * two
    theta = constant(builder, theta, sh)
    freq = pow(builder, theta, f)
    inv_freq = inverse(builder, freq)

    sh = make_shape(builder, seq_len, half_dim)
    inv_freq = broadcast(builder, inv_freq, sh)

    pos = arange(builder, seq_len)
    pos = cast(builder, pos, abi.F32)
    sh = make_shape(builder, seq_len, 1)
    pos = reshape(builder, sh, pos)
    sh = shape(builder, inv_freq)
    pos = broadcast(builder, pos, sh)
    pos = pos * inv_freq
    c = cos(builder, pos)
    s = sin(builder, pos)
    c = concat(builder, 1, c, c)
    s = concat(builder, 1, s, s)
    return c, s


# helpers.rs:195-199
def rotate_half(builder, head_dim, x):
    v = chunk(builder, 3, 2, head_dim // 2, x)
    return concat(builder, 3, -v[1], v[0])


# helpers.rs:201-221
def apply_rope_embedding(builder, pos, head_dim, cos, sin, x):
    sh = shape(builder, x)
    _, _, seq_len, _ = unpack(builder, 4, sh)
    pos = to_nat(builder, pos)
    cos = slice(builder, 0, pos, seq_len, cos)
    sin = slice(builder, 0, pos, seq_len, sin)
    cos = broadcast(builder, cos, sh)
    sin = broadcast(builder, sin, sh)
    rotated_x = rotate_half(builder, head_dim, x)
    return cos * x + sin * rotated_x


# helpers.rs:223-237
def rope(builder, theta, pos, seq_len, head_dim, x):
    pos = to_nat(builder, pos)
    seq_len = to_nat(builder, seq_len)
    c, s = rope_tables(builder, theta, pos + seq_len, head_dim)
    return apply_rope_embedding(builder, pos, head_dim, c, s, x)


# helpers.rs:239-257
def causal_mask(builder, size):
    i = arange(builder, size)
    sh = pack(builder, [size, size])
    i = broadcast(builder, i, sh)
    one = to_nat(builder, 1)
    shr = pack(builder, [size, one])
    j = arange(builder, size)
    j = reshape(builder, shr, j)
    j = broadcast(builder, j, sh)
    mask = lt(builder, j, i)
    mask = cast(builder, mask, abi.F32)
    sh = shape(builder, mask)
    ninf = constant(builder, F32_MIN, sh)
    return mask * ninf


# helpers.rs:259-271
def embeddings(builder, p, x):
    wte = param(builder, p.extend(["weight"]))
    b, s = unpack(builder, 2, shape(builder, x))
    x = reshape(builder, make_shape(builder, b * s), x)
    te = index(builder, 0, x, wte)
    return unsqueeze(builder, 2, 0, te)

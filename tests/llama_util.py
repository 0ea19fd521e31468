"""Shared helpers for the Llama parity tests: a tiny configuration; the seeded parameters and the
decode driver come from the package."""
import importlib

cg = importlib.import_module("catgrad-rs_amd")
llm = importlib.import_module("catgrad-rs_amd.llm")
llama = llm.llama
param_arrays = llm.random_init.llama_params
interpreter = llm.runner.interpreter
CachedRunner = llm.runner.CachedRunner


def tiny_config(**kw):
    c = dict(hidden_size=64, intermediate_size=160, num_hidden_layers=2, num_attention_heads=4,
             num_key_value_heads=2, vocab_size=211, rms_norm_eps=1e-5, rope_theta=500000.0,
             tie_word_embeddings=True)
    c.update(kw)
    return llm.Config(**c)

#!/usr/bin/env python3
"""Writes tests/golden/qwen_moe_full_width.npz: the CPU oracle on one layer of the Qwen-MoE layout at its real
width (hidden 2048, 16 heads of 128, 60 routed experts of 1408 with top-4 routing, shared expert of 5632,
vocabulary cut to 1024), 4 prompts of 16 tokens.  The as-written expert gather costs the oracle minutes at
this width, so its results are kept as vectors:
  f32 parameters:      the KV-cached prefill's last-position logits and tokens, and the logits of one decode
                       step of four rows fed those tokens;
  rounded parameters (what bf16 mode stores): the full-recompute model's logits at every position, the
                       mask of positions exposed to a router near tie (k-th and (k+1)-th router logit closer
                       than 2e-2 of the row's largest; with one layer no attention reads a routed result,
                       so a near tie exposes its own position only), and the same decode step.
Parameters and prompts are rebuilt by the test from the same seeds (tests/model_util.py).

Run from the repository root after `make -C oracle`:  python tests/golden/make_qwen_moe_full_width.py
(nothing of the reference is imported or run)."""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

NEAR_TIE = 2e-2


def setup(MU):
    cfg = MU.qwen_moe_config(hidden_size=2048, num_hidden_layers=1, num_attention_heads=16, num_key_value_heads=16,
                             head_dim=128, vocab_size=1024, num_experts=60, num_experts_per_tok=4,
                             moe_intermediate_size=1408, shared_expert_intermediate_size=5632)
    P = MU.qwen_moe_params(cfg, seed=21, std=0.02)
    # router logits with a spread of a few units (normed rows of 2048 values against N(0, s) weights)
    P["qwen_moe.model.layers.0.mlp.gate.weight"] *= np.float32(0.1)
    prompts = np.random.default_rng(22).integers(0, cfg.vocab_size, (4, 16))
    return cfg, P, prompts


def main():
    import model_util as MU
    import llama_util as U
    cg, llm = U.cg, U.llm
    nn = importlib.import_module("catgrad-rs_amd.nn")
    oracle = cg.Backend(cg.load_library(os.path.join(ROOT, "oracle", "liboracle.so")))
    cfg, P, prompts = setup(MU)

    def cached(params):
        r = U.CachedRunner(oracle, cfg, params, 32, prefill_cls=llm.qwen_moe.QwenMoePrefill,
                           decode_cls=llm.qwen_moe.QwenMoeDecode)
        tok, logits = r.prefill(prompts)
        tok = oracle.to_vec(tok).reshape(-1)
        pre = oracle.numpy(logits)
        _, logits = r.step(tok)
        return tok, pre, oracle.numpy(logits)
    out = {}
    out["f32_tokens"], out["f32_prefill_logits"], out["f32_step_logits"] = cached(P)
    print("f32 done", flush=True)
    R = {k: (llm.random_init.bf16_round(v) if v.ndim >= 2 else v) for k, v in P.items()}
    out["rounded_tokens"], _, out["rounded_step_logits"] = cached(R)
    print("rounded cached done", flush=True)

    class WithRouter(llm.qwen_moe.QwenMoeModel):
        def sort(self):
            i, o = super().sort()
            return i, o + [o[0]] * self.config.num_hidden_layers

        def moe(self, builder, p, x):
            c = self.config
            self._router.append(nn.linear_no_bias(builder, c.hidden_size, c.num_experts, p.extend(["gate"]), x))
            return super().moe(builder, p, x)

        def def_(self, builder, args):
            self._router = []
            return super().def_(builder, args) + self._router
    outs = U.interpreter(oracle, R).run(WithRouter(cfg, prompts.shape[1]).term(),
                                        [oracle.tensor(np.asarray(prompts, np.uint32))])
    out["rounded_logits"] = oracle.numpy(outs[1])
    k = cfg.num_experts_per_tok
    near = np.zeros(prompts.shape, bool)
    for layer in outs[2:]:
        lg = oracle.numpy(layer).reshape(prompts.shape + (cfg.num_experts,)).astype(np.float64)
        srt = np.sort(lg, axis=-1)
        near |= (srt[..., -k] - srt[..., -k - 1]) <= NEAR_TIE * np.abs(lg).max(axis=-1)
    assert cfg.num_hidden_layers == 1
    out["rounded_exposed"] = near
    out["prompts"] = prompts
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "qwen_moe_full_width.npz"), **out)
    print("exposed", out["rounded_exposed"].sum(), "of", near.size)


if __name__ == "__main__":
    main()

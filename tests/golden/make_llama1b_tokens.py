#!/usr/bin/env python3
"""Writes tests/golden/llama1b_f32_tokens.json: the CPU oracle (the restated ndarray backend, f32, one
thread) running the Llama-3.2-1B shape of BASELINE configs[2] - random init N(0, 0.02), seed 0, a
16-token prompt drawn with seed 1 - for 32 greedy steps with the KV-cached terms, the loop of
catgrad-llm/examples/llama/main.rs:114-169.  Per step: the token, the gap between the two largest logits
over the rms of the row (a device token may differ only where that gap is below the f32 bar), the eight
largest logits with their columns, and 64 logits at fixed columns.

Run from the repository root after `make -C oracle`:  python tests/golden/make_llama1b_tokens.py
(about five minutes and 12 GB of memory; nothing of the reference is imported or run)."""
import importlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

STEPS, PROMPT = 32, 16


def main():
    cg = importlib.import_module("catgrad-rs_amd")
    llm = importlib.import_module("catgrad-rs_amd.llm")
    oracle = cg.Backend(cg.load_library(os.path.join(ROOT, "oracle", "liboracle.so")))
    cfg = llm.random_init.llama_1b_config(llm.Config, 16)
    arrays = llm.random_init.llama_params(cfg, seed=0, std=0.02)
    prompt = [int(t) for t in np.random.default_rng(1).integers(0, cfg.vocab_size, PROMPT)]
    runner = llm.CachedRunner(oracle, cfg, arrays, PROMPT + STEPS + 1)
    cols = [int(c) for c in np.random.default_rng(2).integers(0, cfg.vocab_size, 64)]
    tok, logits = runner.prefill(prompt)
    steps = []
    for i in range(STEPS):
        t = int(oracle.to_vec(tok)[0])
        row = np.asarray(oracle.to_vec(logits), np.float32)
        r64 = row.astype(np.float64)
        order = np.argsort(-r64, kind="stable")[:8]
        rms = float(np.sqrt(np.mean(r64 * r64)))
        steps.append({"token": t, "gap_over_rms": float((r64[order[0]] - r64[order[1]]) / rms), "rms": rms,
                      "top8_cols": [int(c) for c in order], "top8": [float(row[c]) for c in order],
                      "sample": [float(row[c]) for c in cols]})
        print(i, t, steps[-1]["gap_over_rms"], flush=True)
        if i + 1 < STEPS:
            tok, logits = runner.step(t)
    out = {"workload": "BASELINE configs[2] shape, 16 layers, f32, llama_params(seed=0, std=0.02), prompt = "
                       "default_rng(1).integers(0, 128256, 16), greedy, KV cache",
           "made_by": "tests/golden/make_llama1b_tokens.py (oracle/ndarray_oracle.cpp)",
           "prompt": prompt, "sample_cols": cols, "steps": steps}
    with open(os.path.join(ROOT, "tests", "golden", "llama1b_f32_tokens.json"), "w") as f:
        json.dump(out, f, indent=1)


if __name__ == "__main__":
    main()

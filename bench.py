#!/usr/bin/env python3
"""bench.py — Llama-3.2-1B-shape decoder (random init) through the native evaluator on one MI355X.

One "step" = one greedy decode token with KV cache at batch 1 after a 512-token prefill
(BASELINE.json configs[2]).  Prints ONE JSON line; `value` is decode tokens/s with all inputs
resident in HBM, `roofline` describes the dominant decode kernel (the weight GEMV, HBM-bound),
`cpu_baseline` times the CPU oracle (a restatement of the single-threaded ndarray backend) on a
bounded sample of the same workload.  Extra keys carry prefill throughput and the GEMM roofline.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the decode GEMV kernels at the default workload (bf16, 16 layers), from two
# rocprofv3 --pmc runs of this file (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter
# read for the 1 GiB peak_copy_kernel in the same run (x2.000 and x1.000); a profiler cannot run
# inside this process, so the figure is carried here and reported only for that workload
PMC_TRAFFIC_BYTES_PER_LAUNCH = {("bf16", 16, "gemv_rowdot_bf16"): 38325390.0}
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}


def llama_1b_config(llm, layers):
    return llm.Config(hidden_size=2048, intermediate_size=8192, num_hidden_layers=layers,
                      num_attention_heads=32, num_key_value_heads=8, vocab_size=128256,
                      rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True)


def matmul_params(cfg):
    h, f, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    kv = h // (cfg.num_attention_heads // cfg.num_key_value_heads)
    per_layer = 2 * h * h + 2 * kv * h + 3 * f * h
    return cfg.num_hidden_layers * per_layer + v * h


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=32)
    ap.add_argument("--warmup", type=int, default=4)
    ap.add_argument("--dtype", choices=["bf16", "f32"], default="bf16")
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--layers", type=int, default=None)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-steps", type=int, default=3)
    ap.add_argument("--workload", choices=["llama", "ops", "qwen_moe", "gemma3"], default="llama",
                    help="ops: the single-op microbenchmarks (one JSON line with a table); qwen_moe / gemma3: "
                         "BASELINE configs[3] / [4] at full shape (--layers to shorten)")
    ap.add_argument("--sync-each-step", action="store_true",
                    help="read every token on the host before starting the next step")
    ap.add_argument("--profile-only", action="store_true",
                    help="skip the CPU baseline and the traced pass (for rocprofv3 runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    cg = importlib.import_module("catgrad-rs_amd")
    llm = importlib.import_module("catgrad-rs_amd.llm")
    import llama_util as U

    lib = cg.load_library()
    if args.workload in ("qwen_moe", "gemma3"):
        mb = importlib.import_module("catgrad-rs_amd.modelbench")
        if args.workload == "qwen_moe":
            rec = mb.run_qwen_moe(lib, layers=args.layers or 24, steps=args.steps, warmup=args.warmup)
        else:
            rec = mb.run_gemma3(lib, layers=args.layers or 26)
        print(json.dumps({"metric": rec.pop("workload"), "n_gpus": 1, "dtype": "bf16", "data": "synthetic", **rec}))
        return
    args.layers = args.layers or 16
    cfg = llama_1b_config(llm, args.layers)
    if args.workload == "ops":
        opbench = importlib.import_module("catgrad-rs_amd.opbench")
        recs = opbench.run_all(lib, iters=max(args.steps, 10))
        print(json.dumps({"metric": "single-op microbenchmarks through the evaluator (BASELINE configs[0], [1])",
                          "n_gpus": 1, "data": "synthetic", "hbm_peak_gbs": HBM_PEAK_GBS,
                          "mfma_peak_tflops": MFMA_PEAK_TFLOPS, "ops": recs}))
        return
    be = cg.Backend(lib, flags=cg.FLAG_BF16 if args.dtype == "bf16" else 0)
    t0 = time.time()
    arrays = U.param_arrays(cfg, seed=0, std=0.02)
    runner = U.CachedRunner(be, cfg, arrays, args.prompt + args.warmup + args.steps + 16)
    be.sync()
    setup_s = time.time() - t0
    prompt = np.random.default_rng(1).integers(0, cfg.vocab_size, args.prompt).astype(np.uint32)

    # ---- prefill (untimed warm-up pass, then one timed pass) ------------------------------
    tok, _ = runner.prefill(prompt)
    be.to_vec(tok)
    be.sync()
    t = time.perf_counter()
    tok, _ = runner.prefill(prompt)
    first = int(be.to_vec(tok)[0])
    be.sync()
    prefill_s = time.perf_counter() - t

    # ---- decode: W warm-up steps, then exactly K timed steps -------------------------------
    # Default loop: the sampled token stays on the device as the next step's input and the host
    # reads it one step behind (cg_tensor_prefetch), so recording and issuing step t+1 overlap
    # the device's work on step t.  --sync-each-step reads every token before the next step
    # starts, like the reference's driver (catgrad-llm/examples/llama/main.rs:114-169).
    def decode(n, tok_tensor):
        toks = []
        if args.sync_each_step:
            token = int(be.to_vec(tok_tensor)[0])
            for _ in range(n):
                tok_tensor, _ = runner.step(token)
                token = int(be.to_vec(tok_tensor)[0])
                toks.append(token)
            return toks, tok_tensor
        prev = tok_tensor
        for _ in range(n):
            cur, _ = runner.step(prev)
            be.prefetch(cur)
            if prev is not tok_tensor:
                toks.append(int(be.to_vec(prev)[0]))
            prev = cur
        toks.append(int(be.to_vec(prev)[0]))
        return toks, prev

    _, tok = decode(args.warmup, tok) if args.warmup else ([], tok)
    be.sync()
    runner.it.backend_calls()
    launches0 = be.stats()["launches"]
    t = time.perf_counter()
    toks, tok = decode(args.steps, tok)
    be.sync()
    decode_s = time.perf_counter() - t
    token = toks[-1]
    calls_per_step = runner.it.backend_calls() / max(args.steps, 1)
    launches_per_step = (be.stats()["launches"] - launches0) / max(args.steps, 1)
    ms_per_step = decode_s / args.steps * 1e3
    value = args.steps / decode_s

    wbytes = 2 if args.dtype == "bf16" else 4
    n_params = matmul_params(cfg)
    t_mid = args.prompt + args.warmup + args.steps / 2
    kv_bytes = 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * 64 * t_mid * 4
    algo_bytes_per_token = n_params * wbytes + kv_bytes

    out = {
        "metric": "decode tokens/sec (Llama-3.2-1B shape, batch 1, KV cache, greedy, 1 GPU)",
        "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: Llama-3.2-1B shape, random init N(0,0.02), "
                               f"{cfg.num_hidden_layers} layers, batch 1, {args.prompt}-token prompt, "
                               "greedy decode with KV cache through the catgrad evaluator; "
                               + ("token read back before every step" if args.sync_each_step else
                                  "token fed back on the device, read by the host one step behind"),
                   "prompt_tokens": args.prompt, "layers": cfg.num_hidden_layers},
        "prefill_tokens_per_s": args.prompt / prefill_s,
        "prefill_ms": prefill_s * 1e3,
        "decode_fraction_of_hbm_roofline": (algo_bytes_per_token * value) / (HBM_PEAK_GBS * 1e9),
        "algorithmic_bytes_per_token": algo_bytes_per_token,
        "backend_calls_per_step": calls_per_step,
        "kernel_launches_per_step": launches_per_step,
        "setup_s": setup_s,
    }

    # ---- what this device gives the simplest code (denominators next to the data-sheet peaks) ----
    out["measured_peaks"] = {"copy_gbs_read_plus_write": be.peak_copy_gbs(1 << 30, 10),
                             "mfma_bf16_tflops": be.peak_mfma_tflops(cg.abi.U32, 20000),
                             "mfma_f32_tflops": be.peak_mfma_tflops(cg.abi.F32, 20000)}

    if not args.profile_only:
        # ---- traced pass: per-kernel durations from events on the backend's own stream ---------
        be.trace(True)
        be.trace_reset()
        n_tr = min(8, max(args.steps, 1))
        for _ in range(n_tr):
            tok, _ = runner.step(token)
            token = int(be.to_vec(tok)[0])
        rep = be.trace_report()
        gemv = "gemv_rowdot_bf16" if args.dtype == "bf16" else "gemv_rowdot_f32"
        if gemv in rep and rep[gemv]["ms"] > 0:
            r = rep[gemv]
            achieved = r["bytes"] / (r["ms"] * 1e-3) / 1e9
            out["roofline"] = {"bound": "hbm", "kernel": gemv, "achieved": achieved, "peak": HBM_PEAK_GBS,
                               "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                               "traffic": PMC_TRAFFIC_BYTES_PER_LAUNCH.get((args.dtype, args.layers, gemv)),
                               "launches_per_step": r["launches"] / n_tr,
                               "avg_us": r["ms"] * 1e3 / r["launches"],
                               "algorithmic_bytes_per_launch": r["bytes"] / r["launches"]}
        total_ms = sum(v["ms"] for v in rep.values()) or 1.0
        out["decode_kernel_time_share"] = {
            k: round(v["ms"] / total_ms, 4)
            for k, v in sorted(rep.items(), key=lambda kv: -kv[1]["ms"])[:8]}
        out["decode_kernel_ms_per_step"] = total_ms / n_tr
        # prefill GEMM roofline
        be.trace_reset()
        tok, _ = runner.prefill(prompt)
        be.to_vec(tok)
        rep = be.trace_report()
        gemm = "gemm_mfma_bf16" if args.dtype == "bf16" else "gemm_mfma_f32"
        if gemm in rep and rep[gemm]["ms"] > 0:
            r = rep[gemm]
            tf = r["flops"] / (r["ms"] * 1e-3) / 1e12
            peak = MFMA_PEAK_TFLOPS[args.dtype]
            out["prefill_gemm_roofline"] = {"bound": "mfma", "kernel": gemm, "achieved": tf, "peak": peak,
                                            "unit": "TFLOP/s", "frac": tf / peak,
                                            "launches": r["launches"], "total_ms": r["ms"]}
        ptotal = sum(v["ms"] for v in rep.values()) or 1.0
        out["prefill_kernel_time_share"] = {
            k: round(v["ms"] / ptotal, 4)
            for k, v in sorted(rep.items(), key=lambda kv: -kv[1]["ms"])[:8]}
        be.trace(False)

    if not args.no_cpu_baseline and not args.profile_only:
        # ---- CPU baseline: the oracle (restated single-threaded ndarray backend), f32, on a
        # bounded sample: KV-cached decode steps after a 16-token prefill (the weights dominate a
        # decode step at any cache length here).
        olib = cg.load_library(os.path.join(ROOT, "oracle", "liboracle.so"))
        obe = cg.Backend(olib)
        cr = U.CachedRunner(obe, cfg, arrays, 64)
        tk, _ = cr.prefill(prompt[:16])
        tkn = int(obe.to_vec(tk)[0])
        t = time.perf_counter()
        for _ in range(args.cpu_steps):
            tk, _ = cr.step(tkn)
            tkn = int(obe.to_vec(tk)[0])
        cpu_s = time.perf_counter() - t
        out["cpu_baseline"] = {
            "value": args.cpu_steps / cpu_s, "unit": "tokens/s", "cores": 1, "kind": "port",
            "host_cores": os.cpu_count(),
            "sample": f"{args.cpu_steps} KV-cached decode steps at cache length 16.. after a 16-token "
                      "prefill, f32, restated ndarray backend (Rust toolchain unavailable), 1 thread"}

    print(json.dumps(out))


if __name__ == "__main__":
    main()

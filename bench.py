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

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}
# HBM bytes per launch of the decode GEMV kernels at the default workload come from two rocprofv3 --pmc
# runs of this file (FETCH_SIZE, WRITE_SIZE; a profiler cannot run inside this process).  Their
# summary, with the commands, is these files; their "traffic_bytes_per_launch" line is read, so the figure
# reported is the one the committed counters show, for the workload they were taken on only.
PMC_SUMMARY = {dt: os.path.join(ROOT, "profiles", f"gemv_rowdot_{dt}_llama1b_decode_pmc.txt") for dt in ("bf16", "f32")}


def pmc_traffic_bytes_per_launch(dtype, layers, kernel):
    """The `traffic_bytes_per_launch[dtype,layers,kernel] = N` line of the PMC summary, or None."""
    key = f"traffic_bytes_per_launch[{dtype},{layers},{kernel}]"
    try:
        for line in open(PMC_SUMMARY[dtype]):
            if key in line:
                return float(line.split("=")[1].split()[0])
    except (OSError, KeyError):
        pass
    return None


def matmul_params(cfg):
    h, f, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    kv = h // (cfg.num_attention_heads // cfg.num_key_value_heads)
    per_layer = 2 * h * h + 2 * kv * h + 3 * f * h
    return cfg.num_hidden_layers * per_layer + v * h


def other_configs(lib, args):
    """The other BASELINE configurations, after the timed region: configs[1] op by op (f32 and bf16
    storage, each with its roofline fraction), configs[0] (the 64x128x256x10 MLP, microseconds per run),
    configs[3] (Qwen-MoE layout) and configs[4] (Gemma-3 shape) at full size; and the bf16 GEMM alone over
    the cubes and the models' product shapes."""
    opbench = importlib.import_module("benchmarks.opbench")
    mb = importlib.import_module("benchmarks.modelbench")
    res = {}
    recs = opbench.run_all(lib, iters=20)
    for dtype in ("f32", "bf16"):
        table = {}
        for r in recs:
            if r["dtype"] != dtype or r["bound"] == "latency":
                continue
            table[r["op"]] = {"bound": r["bound"], "achieved": r["tflops"] if r["bound"] == "mfma" else r["gbs"],
                              "unit": "TFLOP/s" if r["bound"] == "mfma" else "GB/s", "frac": r["frac"],
                              "kernel_us": r["kernel_us"], "wall_us": r["wall_us"]}
        res["ops_" + dtype] = table
    mlp = [r for r in recs if r["bound"] == "latency"]
    if mlp:
        res["mlp_us"] = {"wall_us_per_run": mlp[0]["wall_us"], "kernel_us_per_run": mlp[0]["kernel_us"],
                         "launches": sum(mlp[0]["kernels"].values())}
    sweep = importlib.import_module("benchmarks.gemm_sweep")
    res["gemm_bf16_sweep"] = {r["shape"]: {"achieved": r["tflops"], "unit": "TFLOP/s", "frac": r["frac"], "us": r["us"],
                                           "clock_mhz": r.get("clock_mhz"), "frac_at_clock": r.get("frac_at_clock")}
                              for r in sweep.run(lib, iters=5)}
    q = mb.run_qwen_moe(lib, steps=16, warmup=2)
    res["qwen_moe"] = {"ms_per_step": q["ms_per_step"], "decode_tokens_per_s": q["decode_tokens_per_s"],
                       "prefill_ms": q["prefill_ms"], "prefill_tokens_per_s": q["prefill_tokens_per_s"],
                       "kernel_launches_per_step": q["kernel_launches_per_step"],
                       "roofline_frac_hbm_upper_bound_bytes": q["decode_hbm_fraction_at_upper_bound"],
                       "distinct_experts_per_layer_and_step": q["distinct_experts_per_layer_and_step"],
                       "roofline_frac_hbm": q["decode_hbm_fraction"],
                       "workload": q["workload"]}
    g = mb.run_gemma3(lib)
    res["gemma3"] = {"prefill_ms": g["prefill_ms"], "prefill_tokens_per_s": g["prefill_tokens_per_s"],
                     "tflops_end_to_end": g["matmul_tflops_end_to_end"],
                     "roofline_frac_mfma_end_to_end": g["matmul_tflops_end_to_end"] / MFMA_PEAK_TFLOPS["bf16"],
                     "gemm_tflops": g["gemm_tflops"], "workload": g["workload"]}
    return res


def measure_llama(cg, llm, lib, cfg, arrays, prompt, dtype, args, steps, warmup, peaks=True):
    """Prefill (median of three passes after two warm-up passes), `warmup` untimed and `steps` timed
    KV-cached greedy decode steps, then - unless args.profile_only - a traced pass for the per-kernel
    rooflines.  Returns the record; the backend is released before returning."""
    be = cg.Backend(lib, flags=cg.FLAG_BF16 if dtype == "bf16" else 0)
    t0 = time.time()
    runner = llm.CachedRunner(be, cfg, arrays, args.prompt + warmup + steps + 16)
    be.sync()
    setup_s = time.time() - t0

    for _ in range(2):
        tok, _ = runner.prefill(prompt)
        be.to_vec(tok)
    passes = []
    for _ in range(3):
        be.sync()
        t = time.perf_counter()
        tok, _ = runner.prefill(prompt)
        int(be.to_vec(tok)[0])
        be.sync()
        passes.append(time.perf_counter() - t)
    prefill_s = sorted(passes)[1]

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

    _, tok = decode(warmup, tok) if warmup else ([], tok)
    be.sync()
    runner.it.backend_calls()
    launches0 = be.stats()["launches"]
    t = time.perf_counter()
    toks, tok = decode(steps, tok)
    be.sync()
    decode_s = time.perf_counter() - t
    token = toks[-1]
    calls_per_step = runner.it.backend_calls() / max(steps, 1)
    launches_per_step = (be.stats()["launches"] - launches0) / max(steps, 1)
    value = steps / decode_s

    wbytes = 2 if dtype == "bf16" else 4
    n_params = matmul_params(cfg)
    t_mid = args.prompt + warmup + steps / 2
    kv_bytes = 2 * cfg.num_hidden_layers * cfg.num_key_value_heads * 64 * t_mid * 4
    algo_bytes_per_token = n_params * wbytes + kv_bytes
    out = {
        "value": value, "ms_per_step": decode_s / steps * 1e3, "steps": steps, "warmup": warmup,
        "prefill_tokens_per_s": args.prompt / prefill_s,
        "prefill_ms": prefill_s * 1e3,
        "decode_fraction_of_hbm_roofline": (algo_bytes_per_token * value) / (HBM_PEAK_GBS * 1e9),
        "algorithmic_bytes_per_token": algo_bytes_per_token,
        "backend_calls_per_step": calls_per_step,
        "kernel_launches_per_step": launches_per_step,
        "setup_s": setup_s,
    }
    if peaks:
        # what this device gives the simplest code (denominators next to the data-sheet peaks)
        out["measured_peaks"] = {"copy_gbs_read_plus_write": be.peak_copy_gbs(1 << 30, 10),
                                 "mfma_bf16_tflops": be.peak_mfma_tflops(cg.abi.U32, 20000),
                                 "mfma_f32_tflops": be.peak_mfma_tflops(cg.abi.F32, 20000)}
        # the shader clock (read inside the kernels) under the bare MFMA loop and under the bf16 GEMM: the
        # data-sheet 2.5 PFLOP/s is 2400 MHz; a GEMM is clocked lower by the power limit
        loop_tf, loop_mhz = be.peak_gemm_clock(0, 0, 0, 2)
        g4_tf, g4_mhz = be.peak_gemm_clock(4096, 4096, 4096, 5)
        g8_tf, g8_mhz = be.peak_gemm_clock(8192, 8192, 8192, 3)
        out["measured_peaks"]["shader_clock_mhz"] = {
            "data_sheet": 2400, "mfma_loop": loop_mhz, "gemm_bf16_4096": g4_mhz, "gemm_bf16_8192": g8_mhz,
            "gemm_bf16_4096_tflops": g4_tf, "gemm_bf16_8192_tflops": g8_tf,
            "gemm_bf16_8192_frac_of_mfma_peak_at_its_clock": g8_tf / (MFMA_PEAK_TFLOPS["bf16"] * g8_mhz / 2400.0)
            if g8_mhz else None}
    if not args.profile_only:
        # ---- traced pass: per-kernel durations from events on the backend's own stream ---------
        be.trace(True)
        be.trace_reset()
        n_tr = min(8, max(steps, 1))
        for _ in range(n_tr):
            tok, _ = runner.step(token)
            token = int(be.to_vec(tok)[0])
        rep = be.trace_report()
        gemv = "gemv_rowdot_bf16" if dtype == "bf16" else "gemv_rowdot_f32"
        if gemv in rep and rep[gemv]["ms"] > 0:
            r = rep[gemv]
            achieved = r["bytes"] / (r["ms"] * 1e-3) / 1e9
            out["roofline"] = {"bound": "hbm", "kernel": gemv, "achieved": achieved, "peak": HBM_PEAK_GBS,
                               "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                               "traffic": pmc_traffic_bytes_per_launch(dtype, cfg.num_hidden_layers, gemv),
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
        gemm = "gemm_mfma_bf16" if dtype == "bf16" else "gemm_mfma_f32"
        if gemm in rep and rep[gemm]["ms"] > 0:
            r = rep[gemm]
            tf = r["flops"] / (r["ms"] * 1e-3) / 1e12
            peak = MFMA_PEAK_TFLOPS[dtype]
            out["prefill_gemm_roofline"] = {"bound": "mfma", "kernel": gemm, "achieved": tf, "peak": peak,
                                            "unit": "TFLOP/s", "frac": tf / peak,
                                            "launches": r["launches"], "total_ms": r["ms"]}
        ptotal = sum(v["ms"] for v in rep.values()) or 1.0
        out["prefill_kernel_time_share"] = {
            k: round(v["ms"] / ptotal, 4)
            for k, v in sorted(rep.items(), key=lambda kv: -kv[1]["ms"])[:8]}
        be.trace(False)
    del runner, tok
    be.close()
    return out


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
                    help="skip the CPU baseline, the traced pass and the other configurations (for rocprofv3 runs)")
    ap.add_argument("--no-f32", action="store_true", help="skip the f32-mode pass of the same workload")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the other BASELINE configurations (ops, MLP, Qwen-MoE, Gemma-3) after the timed region")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (no collectives, no sharding); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    cg = importlib.import_module("catgrad-rs_amd")
    llm = importlib.import_module("catgrad-rs_amd.llm")

    lib = cg.load_library()
    if args.workload in ("qwen_moe", "gemma3"):
        mb = importlib.import_module("benchmarks.modelbench")
        if args.workload == "qwen_moe":
            rec = mb.run_qwen_moe(lib, layers=args.layers or 24, steps=args.steps, warmup=args.warmup, count_experts=not args.profile_only)
        else:
            rec = mb.run_gemma3(lib, layers=args.layers or 26)
        print(json.dumps({"metric": rec.pop("workload"), "n_gpus": 1, "dtype": "bf16", "data": "synthetic", **rec}))
        return
    args.layers = args.layers or 16
    cfg = llm.random_init.llama_1b_config(llm.Config, args.layers)
    if args.workload == "ops":
        opbench = importlib.import_module("benchmarks.opbench")
        recs = opbench.run_all(lib, iters=max(args.steps, 10))
        print(json.dumps({"metric": "single-op microbenchmarks through the evaluator (BASELINE configs[0], [1])",
                          "n_gpus": 1, "data": "synthetic", "hbm_peak_gbs": HBM_PEAK_GBS,
                          "mfma_peak_tflops": MFMA_PEAK_TFLOPS, "ops": recs}))
        return
    arrays = llm.random_init.llama_params(cfg, seed=0, std=0.02)
    prompt = np.random.default_rng(1).integers(0, cfg.vocab_size, args.prompt).astype(np.uint32)
    rec = measure_llama(cg, llm, lib, cfg, arrays, prompt, args.dtype, args, args.steps, args.warmup)

    out = {
        "metric": "decode tokens/sec (Llama-3.2-1B shape, batch 1, KV cache, greedy, 1 GPU)",
        "value": rec.pop("value"), "unit": "tokens/s", "n_gpus": 1, "steps": rec.pop("steps"),
        "warmup": rec.pop("warmup"),
        "ms_per_step": rec.pop("ms_per_step"), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "BASELINE configs[2]: Llama-3.2-1B shape, random init N(0,0.02), "
                               f"{cfg.num_hidden_layers} layers, batch 1, {args.prompt}-token prompt, "
                               "greedy decode with KV cache through the catgrad evaluator; "
                               + ("token read back before every step" if args.sync_each_step else
                                  "token fed back on the device, read by the host one step behind"),
                   "prompt_tokens": args.prompt, "layers": cfg.num_hidden_layers},
    }
    out.update(rec)

    if args.dtype == "bf16" and not args.profile_only and not args.no_f32:
        # the same workload in f32 mode - the reference's own arithmetic - after the timed region
        f = measure_llama(cg, llm, lib, cfg, arrays, prompt, "f32", args, min(args.steps, 16), min(args.warmup, 2),
                          peaks=False)
        out["llama_f32"] = {"decode_tokens_per_s": f["value"], "ms_per_step": f["ms_per_step"], "steps": f["steps"],
                            "prefill_ms": f["prefill_ms"], "prefill_tokens_per_s": f["prefill_tokens_per_s"],
                            "roofline": f.get("roofline"), "prefill_gemm_roofline": f.get("prefill_gemm_roofline"),
                            "decode_fraction_of_hbm_roofline": f["decode_fraction_of_hbm_roofline"],
                            "kernel_launches_per_step": f["kernel_launches_per_step"]}

    if not args.no_cpu_baseline and not args.profile_only:
        # ---- CPU baseline: the oracle (restated single-threaded ndarray backend), f32, on a
        # bounded sample: KV-cached decode steps after a 16-token prefill (the weights dominate a
        # decode step at any cache length here).
        olib = cg.load_library(os.path.join(ROOT, "oracle", "liboracle.so"))
        obe = cg.Backend(olib)
        cr = llm.CachedRunner(obe, cfg, arrays, 64)
        t = time.perf_counter()
        tk, lg = cr.prefill(prompt[:16])
        tkn = int(obe.to_vec(tk)[0])
        cpu_prefill_s = time.perf_counter() - t
        o_toks, o_logits = [tkn], [obe.to_vec(lg)]
        t = time.perf_counter()
        for _ in range(args.cpu_steps):
            tk, lg = cr.step(tkn)
            tkn = int(obe.to_vec(tk)[0])
            o_toks.append(tkn)
            o_logits.append(obe.to_vec(lg))
        cpu_s = time.perf_counter() - t
        out["cpu_baseline"] = {
            "value": args.cpu_steps / cpu_s, "unit": "tokens/s", "cores": 1, "kind": "port",
            "host_cores": os.cpu_count(),
            "prefill_tokens_per_s": 16 / cpu_prefill_s,
            "sample": f"{args.cpu_steps} KV-cached decode steps at cache length 16.. after a 16-token "
                      "prefill (timed as prefill_tokens_per_s), f32, restated ndarray backend (Rust "
                      "toolchain unavailable), 1 thread"}
        del cr, tk, lg
        obe.close()
        # ---- the same sample on the device in f32, compared with what the oracle just computed
        # (outside every timed region): identical tokens and logits within rel 1e-4, per element
        # against max(|logit|, rms of the row)
        fbe = cg.Backend(lib)
        gr = llm.CachedRunner(fbe, cfg, arrays, 64)
        g_toks, g_logits = gr.generate(prompt[:16], args.cpu_steps + 1)
        worst, margin = 0.0, None
        for a, b_ in zip(o_logits, g_logits):
            a64 = a.astype(np.float64)
            floor = np.sqrt(np.mean(a64 * a64))
            worst = max(worst, float(np.max(np.abs(a64 - b_) / np.maximum(np.abs(a64), floor))))
            top = np.sort(a64)[-2:]
            m = float((top[1] - top[0]) / floor)
            margin = m if margin is None else min(margin, m)
        out["parity_checked"] = bool(worst <= 1e-4 and g_toks == o_toks)
        out["parity"] = {"against": "the oracle's logits and tokens on the CPU-baseline sample (full shape, f32)",
                         "positions": len(o_logits), "max_rel_err": worst, "tolerance": 1e-4,
                         "tokens_identical": g_toks == o_toks, "min_top1_top2_margin_over_rms": margin}
        del gr
        fbe.close()

    if not args.profile_only and not args.no_extras:
        out.update(other_configs(lib, args))

    print(json.dumps(out))


if __name__ == "__main__":
    main()

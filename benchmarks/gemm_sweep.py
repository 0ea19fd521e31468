"""bf16 GEMM sweep through the C ABI: y = x . W^T with x [M, K] and W [N, K] stored as bf16 (the layout
of every linear layer, nn/mod.rs:174-199), f32 accumulation, f32 result.  One matmul per launch, timed
with the backend's per-launch events.  Run as a script it prints one line per shape; `run(lib)` returns
the records (bench.py reports them)."""
import importlib
import sys
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
cg = importlib.import_module("catgrad-rs_amd")

MFMA_PEAK_BF16_TFLOPS = 2500.0
# (batch, M, N, K): the cubes, BASELINE configs[1]'s bmm, the products of a 512-token Llama-3.2-1B prefill
# (q/k/v, gate or up, o_proj; down_proj is 512 x 2048 x 8192), and Gemma-3's gate / up at batch 8 x 2048
SHAPES = [(1, 8192, 8192, 8192), (1, 4096, 4096, 4096), (8, 1024, 1024, 1024), (1, 512, 3072, 2048),
          (1, 512, 8192, 2048), (1, 512, 2048, 2048), (1, 512, 2048, 8192), (1, 16384, 6912, 1152),
          (1, 16384, 1152, 6912)]


def run(lib, shapes=SHAPES, iters=10, k_major=False):
    be = cg.Backend(lib, flags=cg.FLAG_BF16)
    g = np.random.default_rng(0)
    out = []
    for b, m, n, k in shapes:
        x = be.tensor(g.standard_normal((b, m, k), dtype=np.float32))
        if k_major:                                      # the right operand of a product of two activations: [b, K, N] as stored
            wt = be.tensor(g.standard_normal((b, k, n), dtype=np.float32))
        else:
            w = be.tensor(g.standard_normal((b, n, k), dtype=np.float32))
            wt = be.transpose(w, 1, 2)                   # [b, K, N] view, unit stride along k
        be.realize(be.matmul(x, wt))
        be.sync()
        be.trace(True)
        be.trace_reset()
        for _ in range(iters):
            be.realize(be.matmul(x, wt))
        be.sync()
        rep = be.trace_report()
        be.trace(False)
        ms = sum(v["ms"] for v in rep.values()) / iters
        tf = 2.0 * b * m * n * k / (ms * 1e-3) / 1e12
        rec = {"shape": f"{b}x{m}x{n}x{k}", "us": ms * 1e3, "tflops": tf, "frac": tf / MFMA_PEAK_BF16_TFLOPS,
               "kernels": {name: v["launches"] // iters for name, v in rep.items()}}
        if b == 1 and m % 128 == 0 and n % 128 == 0 and k % 64 == 0 and not k_major:
            # the same product through the clock probe: the shader clock its main loop ran at (the data-sheet
            # peak is 2400 MHz) and the rate as a fraction of the matrix cores' peak at that clock
            ptf, mhz = be.peak_gemm_clock(m, n, k, iters)
            if mhz:
                rec.update(clock_mhz=mhz, frac_at_clock=tf / (MFMA_PEAK_BF16_TFLOPS * mhz / 2400.0))
        out.append(rec)
        del x, wt
    be.close()
    return out


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("--shapes", default=None, help="comma-separated BxMxNxK list (default: the whole sweep)")
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--k-major", action="store_true", help="B stored [K, N] (unit stride along n) instead of [N, K]")
    a = ap.parse_args()
    shapes = SHAPES if not a.shapes else [tuple(int(v) for v in s.split("x")) for s in a.shapes.split(",")]
    for r in run(cg.load_library(), shapes, a.iters, a.k_major):
        clk = f"  clock {r['clock_mhz']:5.0f} MHz -> {100 * r['frac_at_clock']:5.1f} % at that clock" if "clock_mhz" in r else ""
        print(f"{r['shape']:>22s} {r['us']:9.1f} us {r['tflops']:8.1f} TFLOP/s  {100 * r['frac']:5.1f} % of 2.5 PFLOP/s{clk}  {r['kernels']}",
              flush=True)

"""Single-op microbenchmarks through the native evaluator (BASELINE.json configs[0] and [1]).

Every case builds a term holding one op (or one stdlib definition), keeps its inputs resident on
the device, runs it `iters` times through `Interpreter.run`, and reports
  * wall time per run between two stream waits (evaluator + launch + kernel, pipelined), and
  * kernel time from the backend's own start/stop events per launch,
next to the algorithmic bytes / flops of the op (inputs read once, output written once; a
broadcast operand counts at its own size, not at the broadcast size).
"""
import time

import numpy as np

import importlib

cg = importlib.import_module("catgrad-rs_amd")
abi, lang, nn = cg.abi, cg.lang, cg.nn
Interpreter, Parameters, stdlib = cg.Interpreter, cg.Parameters, cg.stdlib

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "f32": 157.3}


class _Fn(lang.Module):
    def __init__(self, name, n_in, n_out, fn):
        self.name, self.n_in, self.n_out, self.fn = name, n_in, n_out, fn

    def path(self):
        return lang.path(["opbench", self.name])

    def sort(self):
        return [lang.TENSOR] * self.n_in, [lang.TENSOR] * self.n_out

    def def_(self, builder, args):
        out = self.fn(builder, *args)
        return list(out) if isinstance(out, (list, tuple)) else [out]


def _softmax(b, x):
    return nn.softmax(b, x)


def _bcast_add(b, x, y):
    return x + lang.broadcast(b, y, lang.shape(b, x))


def _transpose_materialised(b, x):
    # the reference's transpose is a lazy axis swap; the reshape forces the row-major result
    d0, d1, d2 = lang.unpack(b, 3, lang.shape(b, x))
    return lang.reshape(b, lang.make_shape(b, d0, d2 * d1), lang.transpose(b, 1, 2, x))


def _mlp(b, x, w1, w2):
    h = nn.sigmoid(b, lang.matmul(b, x, w1))
    return lang.matmul(b, h, w2)


def cases(dtype, scale=1):
    """(name, fn, inputs, algorithmic bytes, flops).  `scale` divides the big extents (tests)."""
    g = np.random.default_rng(2)
    es = 2 if dtype == "bf16" else 4     # storage bytes of an uploaded rank>=2 f32 tensor
    n = 4096 // scale
    nb, nm = 8, 1024 // scale
    rows, tab, width = 4096 // scale, 32000 // scale, 2048 // scale

    def rnd(*shape):
        return g.standard_normal(shape, dtype=np.float32)
    out = []
    a, bm = rnd(nb, nm, nm), rnd(nb, nm, nm)
    out.append(("bmm", lang.matmul, [a, bm], 2 * a.size * es + a.size * 4, 2.0 * nb * nm ** 3))
    x, y = rnd(n, n), rnd(n)
    out.append(("broadcast_add", _bcast_add, [x, y], x.size * es + y.size * 4 + x.size * 4, 0))
    out.append(("softmax", _softmax, [x], x.size * es + x.size * 4, 0))
    out.append(("sum", lang.sum, [x], x.size * es + n * 4, 0))
    out.append(("max", lang.max, [x], x.size * es + n * 4, 0))
    out.append(("argmax", lang.argmax, [x], x.size * es + n * 4, 0))
    t = rnd(64, 512 // scale, 512 // scale)
    out.append(("transpose", _transpose_materialised, [t], t.size * es + t.size * 4, 0))
    table = rnd(tab, width)
    ids = g.integers(0, tab, rows).astype(np.uint32)
    out.append(("gather", lambda b, tb, iv: lang.index(b, 0, iv, tb), [table, ids],
                rows * width * (es + 4) + rows * 4, 0))
    return out


def mlp_case():
    """hidden.rs-shaped MLP: x [64,128] U[-1,1]; W1 [128,256], W2 [256,10] ~ N(0, 0.05); seed 0."""
    g = np.random.default_rng(0)
    x = g.uniform(-1, 1, (64, 128)).astype(np.float32)
    w1 = (g.standard_normal((128, 256)) * 0.05).astype(np.float32)
    w2 = (g.standard_normal((256, 10)) * 0.05).astype(np.float32)
    return ("mlp_64x128x256x10", _mlp, [x, w1, w2], 0, 2.0 * 64 * 128 * 256 + 2.0 * 64 * 256 * 10)


ROTATE_BYTES = 512 << 20   # twice the 256 MB memory-side cache


def run_case(be, case, iters=50, warmup=5):
    """Every iteration reads another copy of the inputs and keeps its result alive until as many more have
    been made, so that consecutive launches touch distinct memory: enough copies for inputs + results to
    exceed twice the memory-side cache (the figures are HBM figures, not cache figures)."""
    name, fn, arrays, nbytes, flops = case
    it = Interpreter(be, stdlib(), Parameters())
    term = _Fn(name, len(arrays), 1, fn).term()
    working_set = sum(a.nbytes for a in arrays) + max(arrays[0].nbytes, 1)
    copies = 1 if not nbytes else int(min(16, max(2, -(-ROTATE_BYTES // working_set))))
    sets = [[be.tensor(a) for a in arrays] for _ in range(copies)]
    for args in sets:
        for a in args:
            be.realize(a)
    ring = [None] * copies

    def once(i):
        r = it.run(term, sets[i % copies])[0]
        be.realize(r)
        ring[i % copies] = r
    for i in range(max(warmup, copies)):
        once(i)
    be.sync()
    t = time.perf_counter()
    for i in range(iters):
        once(i)
    be.sync()
    wall_us = (time.perf_counter() - t) / iters * 1e6
    be.trace(True)
    be.trace_reset()
    n_tr = min(iters, 20)
    for i in range(n_tr):
        once(i)
    be.sync()
    rep = be.trace_report()
    be.trace(False)
    kern_us = sum(v["ms"] for v in rep.values()) * 1e3 / n_tr
    rec = {"op": name, "wall_us": wall_us, "kernel_us": kern_us, "input_copies_rotated": copies,
           "kernels": {k: v["launches"] // n_tr for k, v in rep.items()}}
    if flops and nbytes:
        rec.update(bound="mfma", algorithmic_flops=flops, tflops=flops / (kern_us * 1e-6) / 1e12)
    elif nbytes:
        rec.update(bound="hbm", algorithmic_bytes=nbytes, gbs=nbytes / (kern_us * 1e-6) / 1e9)
    else:
        rec.update(bound="latency", algorithmic_flops=flops)
    return rec


def run_all(lib, dtypes=("f32", "bf16"), iters=50):
    out = []
    for dtype in dtypes:
        be = abi.Backend(lib, flags=abi.FLAG_BF16 if dtype == "bf16" else 0)
        for case in cases(dtype):
            rec = run_case(be, case, iters)
            rec["dtype"] = dtype
            if rec["bound"] == "hbm":
                rec["frac"] = rec["gbs"] / HBM_PEAK_GBS
            elif rec["bound"] == "mfma":
                rec["frac"] = rec["tflops"] / MFMA_PEAK_TFLOPS[dtype]
            out.append(rec)
        if dtype == "f32":
            rec = run_case(be, mlp_case(), iters=200, warmup=20)
            rec["dtype"] = dtype
            out.append(rec)
            # a plain 16-byte copy of 1 GiB (peak_copy_kernel): what this device gives a read + write stream, and
            # the launch of known size that calibrates FETCH_SIZE / WRITE_SIZE when this runs under rocprofv3
            out.append({"op": "copy_1GiB", "dtype": dtype, "bound": "hbm", "gbs": be.peak_copy_gbs(1 << 30, 5),
                        "algorithmic_bytes": 2 << 30, "kernels": {"peak_copy_kernel": 1}, "input_copies_rotated": 1,
                        "kernel_us": 0.0, "wall_us": 0.0})
            out[-1]["frac"] = out[-1]["gbs"] / HBM_PEAK_GBS
            out[-1]["kernel_us"] = out[-1]["algorithmic_bytes"] / out[-1]["gbs"] / 1e3
        be.close()
    return out

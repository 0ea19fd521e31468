"""The single-op cases of BASELINE.json configs[1] at their full sizes: HIP against the oracle on
the same seeded inputs (bit-exact for transpose / gather / argmax, rel 1e-4 f32 and 2e-2 bf16
otherwise) plus size-independent properties."""
import importlib

import numpy as np
import pytest

import vectors

opbench = importlib.import_module("benchmarks.opbench")
EXACT = {"transpose", "gather", "argmax"}


def bf16_round(a):
    u = a.view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)


def test_cases_shapes_on_oracle(oracle):
    """Reduced extents (1/8): every case evaluates on the oracle and obeys its invariants."""
    for name, fn, arrays, _, _ in opbench.cases("f32", scale=8):
        (out,) = vectors.run(oracle, fn, 1, *arrays)
        if name == "softmax":
            assert np.allclose(out.sum(-1), 1, atol=1e-5)
        if name == "transpose":
            assert np.array_equal(out.reshape(64, 64, 64), arrays[0].transpose(0, 2, 1))
        if name == "gather":
            assert np.array_equal(out, arrays[0][arrays[1]])
        if name == "bmm":
            assert np.allclose(out, np.matmul(arrays[0].astype(np.float64), arrays[1].astype(np.float64)),
                               rtol=1e-4, atol=1e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_full_size_ops_match_oracle(oracle, hip, hip_bf16, dtype):
    dev = hip if dtype == "f32" else hip_bf16
    for name, fn, arrays, _, _ in opbench.cases(dtype):
        ref_in = [bf16_round(a) if (dtype == "bf16" and a.dtype == np.float32 and a.ndim >= 2) else a
                  for a in arrays]
        (ref,) = vectors.run(oracle, fn, 1, *ref_in)
        (got,) = vectors.run(dev, fn, 1, *arrays)
        assert got.shape == ref.shape, name
        if name in EXACT:
            assert np.array_equal(got, ref), name
        else:
            tol = 2e-2 if dtype == "bf16" else 1e-4
            scale = np.abs(ref).max()
            assert np.max(np.abs(got - ref)) <= tol * scale, (name, np.max(np.abs(got - ref)), scale)
        if name == "softmax":
            assert np.allclose(got.sum(-1), 1, atol=1e-4)
        if name == "max":
            assert np.array_equal(got[:, 0], ref_in[0].max(-1))          # max is exact in any order
        if name == "transpose":
            assert np.array_equal(got.reshape(64, 512, 512), ref_in[0].transpose(0, 2, 1))
        if name == "gather":
            assert np.array_equal(got, ref_in[0][arrays[1]])


@pytest.mark.gpu
def test_mlp_config0(oracle, hip):
    name, fn, arrays, _, _ = opbench.mlp_case()
    (ref,) = vectors.run(oracle, fn, 1, *arrays)
    (got,) = vectors.run(hip, fn, 1, *arrays)
    x, w1, w2 = (a.astype(np.float64) for a in arrays)
    expect = (1 / (1 + np.exp(-(x @ w1)))) @ w2
    assert np.allclose(ref, expect, rtol=1e-4, atol=1e-6)
    assert np.allclose(got, ref, rtol=1e-4, atol=1e-6)


@pytest.mark.gpu
def test_opbench_runs(hip):
    """The benchmark driver itself, on small extents."""
    for case in opbench.cases("f32", scale=8):
        rec = opbench.run_case(hip, case, iters=3, warmup=1)
        assert rec["kernel_us"] > 0 and rec["wall_us"] > 0, rec


@pytest.mark.gpu
def test_peak_probes(hip_bf16):
    """The measured denominators bench.py prints: a copy rate, the MFMA issue rates, and the shader clock read
    inside the bare MFMA loop and inside the bf16 GEMM (a GEMM draws more power and may be clocked lower, never
    higher than the data sheet's 2400 MHz by more than the boost margin)."""
    be = hip_bf16
    assert 500 < be.peak_copy_gbs(1 << 28, 3) < 8000
    assert 100 < be.peak_mfma_tflops(iters=2000) < 2600
    loop_tf, loop_mhz = be.peak_gemm_clock(0, 0, 0, 1)
    tf, mhz = be.peak_gemm_clock(2048, 2048, 2048, 3)
    assert 100 < loop_tf < 2600 and 50 < tf < 2600
    assert 500 < loop_mhz < 2700 and 500 < mhz < 2700
    with pytest.raises(vectors.cg.abi.BackendPanic):
        be.peak_gemm_clock(100, 128, 64, 1)      # m not a multiple of 128

"""One layer each of the Qwen-MoE layout (BASELINE configs[3]) and of Gemma-3 (configs[4]) at their real
widths, HIP against the oracle: the kernel instantiations the benchmarks run - the expert-major routed
GEMM at E = 60 / F = 1408 / H = 2048, one-query attention at d = 128 over four rows, the few-row
products against 2048- and 5632-wide matrices, attention at d = 256 over 2048 positions with a window of
512 (dead tiles at real tile boundaries) - at the stated bars (f32 1e-4, bf16 2e-2).  Vocabularies are cut
to 1024 rows: lm_head at full height is the Llama tests' business."""
import numpy as np
import pytest

import llama_util as U
import model_util as MU
import parity

cg, llm = U.cg, U.llm
pytestmark = pytest.mark.gpu


def rounded(P):
    return {k: (llm.random_init.bf16_round(v) if v.ndim >= 2 else v) for k, v in P.items()}


@pytest.fixture(scope="module")
def qwen_full():
    """Configuration, parameters and prompts as tests/golden/make_qwen_moe_full_width.py builds them, and the
    oracle's results it wrote (the as-written expert gather costs the oracle minutes at this width)."""
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location("make_qwen_moe_full_width",
                                                  os.path.join(here, "golden", "make_qwen_moe_full_width.py"))
    mk = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mk)
    cfg, P, prompts = mk.setup(MU)
    gold = np.load(os.path.join(here, "golden", "qwen_moe_full_width.npz"))
    assert np.array_equal(gold["prompts"], prompts)
    return cfg, P, prompts, gold


def qwen_runner(be, cfg, P):
    return U.CachedRunner(be, cfg, P, 32, prefill_cls=llm.qwen_moe.QwenMoePrefill, decode_cls=llm.qwen_moe.QwenMoeDecode)


def test_qwen_moe_full_width_f32(hip, qwen_full):
    """4 x 16-token prompts and one decode step of four rows, f32, through the KV-cached terms."""
    cfg, P, prompts, gold = qwen_full
    g = qwen_runner(hip, cfg, P)
    gt, gl = g.prefill(prompts)
    parity.assert_f32(gold["f32_prefill_logits"], hip.numpy(gl), "prefill, last positions")
    tok = gold["f32_tokens"]
    gaps = parity.top2_gap_over_max(gold["f32_prefill_logits"])
    same = hip.to_vec(gt).reshape(-1) == tok
    assert np.all(same | (gaps <= 2 * parity.RTOL_F32)), (tok, hip.to_vec(gt), gaps)
    _, gl = g.step(tok)
    parity.assert_f32(gold["f32_step_logits"], hip.numpy(gl), "decode step of four rows")


def test_qwen_moe_full_width_bf16(hip_bf16, qwen_full):
    """The same 64 tokens in bf16 mode through the full-recompute model (every position's logits): the routed
    experts run expert-major on the matrix cores.  Rows are held to 2e-2 except where a router near tie
    (found on the oracle) lets top-k choose another expert; then one decode step of four rows."""
    cfg, P, prompts, gold = qwen_full
    exposed = gold["rounded_exposed"]
    hip_bf16.launch_counts(reset=True)
    it = U.interpreter(hip_bf16, P)
    _, gl = it.run(llm.qwen_moe.QwenMoeModel(cfg, prompts.shape[1]).term(), [hip_bf16.tensor(np.asarray(prompts, np.uint32))])
    gl = hip_bf16.numpy(gl)
    counts = hip_bf16.launch_counts(reset=True)
    assert counts.get("gemm_experts_bf16") == 2, counts          # gate+up, then down_proj, expert-major
    err = parity.per_row_bf16(gold["rounded_logits"], gl).reshape(prompts.shape)
    over = err > parity.RTOL_BF16
    assert not (over & ~exposed).any(), (np.argwhere(over & ~exposed)[:5], err[over & ~exposed][:5])
    assert (~over).mean() >= 0.75, "most tokens must meet the bar outright"
    # a decode step of four rows after the cached prefill, fed the oracle's tokens
    g = qwen_runner(hip_bf16, cfg, P)
    g.prefill(prompts)
    hip_bf16.launch_counts(reset=True)
    _, gl = g.step(gold["rounded_tokens"])
    e = parity.per_row_bf16(gold["rounded_step_logits"], hip_bf16.numpy(gl))
    assert np.all((e <= parity.RTOL_BF16) | exposed[:, -1]), e
    # the launches of that step: eight per layer - q/k/v (with the input norm), attention, o_proj + residual,
    # the shared expert's gate * up with the router and its gate riding along (each reader of the post-attention
    # norm computes it itself), the shared down_proj, the routed experts' two stages (the first makes the router's
    # softmax and top-k), the weighted sum - plus embedding rows, lm_head (with the final norm) and argmax
    # (counted on a second step: the first one after a prefill moves the caches to storage with room to grow)
    hip_bf16.launch_counts(reset=True)
    tok, _ = g.step(gold["rounded_tokens"])
    hip_bf16.to_vec(tok)
    counts = hip_bf16.launch_counts(reset=True)
    assert counts.get("softmax_topk", 0) == 0 and counts.get("rmsnorm_fused", 0) == 0, counts
    assert counts.get("gemv_experts_bf16") == 2 * cfg.num_hidden_layers and counts.get("row_scaled_sum") == cfg.num_hidden_layers, counts
    assert sum(counts.values()) == 8 * cfg.num_hidden_layers + 3, counts


@pytest.fixture(scope="module")
def gemma_full():
    cfg = MU.gemma_config(hidden_size=1152, intermediate_size=6912, num_hidden_layers=2, num_attention_heads=4,
                          num_key_value_heads=1, head_dim=256, vocab_size=1024, sliding_window=512,
                          sliding_window_pattern=2)          # layer 0 local (window 512), layer 1 global
    P = MU.gemma_params(cfg, seed=23, std=0.02)
    ids = np.random.default_rng(24).integers(0, cfg.vocab_size, (1, 2048))
    return cfg, P, ids


@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_gemma3_full_width(oracle, hip, hip_bf16, gemma_full, mode):
    """2048 positions through one local and one global layer; logits of every position."""
    cfg, P, ids = gemma_full
    model = llm.gemma3.Gemma3Model(cfg, ids.shape[1])
    dev = hip if mode == "f32" else hip_bf16
    P_ref = rounded(P) if mode == "bf16" else P
    _, rl = U.interpreter(oracle, P_ref).run(model.term(), [oracle.tensor(np.asarray(ids, np.uint32))])
    rl = oracle.numpy(rl)
    dev.launch_counts(reset=True)
    _, gl = U.interpreter(dev, P).run(model.term(), [dev.tensor(np.asarray(ids, np.uint32))])
    gl = dev.numpy(gl)
    counts = dev.launch_counts(reset=True)
    assert counts.get("attn_prefill") == cfg.num_hidden_layers, counts
    # q and k are normed per head by the launch that rotates them (one per layer for both): what is left of the
    # norms is the input norm of the first layer, two sandwich pairs per layer and the final norm
    assert counts.get("rope_fused") == cfg.num_hidden_layers, counts
    assert counts.get("rmsnorm_fused") <= 2 * cfg.num_hidden_layers + 2, counts
    parity.assert_logits(rl, gl, mode, "Gemma-3 at full width")

"""Qwen-MoE-layout and Gemma-3 decoders at reduced shapes (BASELINE configs 4 and 5): the oracle
against independent numpy statements of the two build-authored pieces (top-k routed experts with
a gated shared expert; sliding-window mask), then HIP vs oracle."""
import numpy as np
import pytest

import llama_util as U
import model_util as MU
import parity

cg, llm = U.cg, U.llm


def run_model(be, module, arrays, ids):
    it = U.interpreter(be, arrays)
    tok, logits = it.run(module.term(), [be.tensor(np.asarray(ids, np.uint32))])
    return be.numpy(tok), be.numpy(logits)


def test_moe_block_matches_numpy(oracle):
    """The routed + shared expert block against a direct numpy statement of the same maths."""
    cfg = MU.qwen_moe_config(num_hidden_layers=1)
    P = MU.qwen_moe_params(cfg, seed=3, std=0.3)
    model = llm.qwen_moe.QwenMoeModel(cfg, 8)
    g = np.random.default_rng(4)
    x = g.standard_normal((1, 6, cfg.hidden_size)).astype(np.float32)
    pre = "qwen_moe.model.layers.0.mlp."

    import vectors
    (y,) = vectors.run(oracle, lambda b, v: model.moe(b, vectors.lang.path(["qwen_moe", "model", "layers", 0, "mlp"]), v),
                       1, x, params={k: v for k, v in P.items() if k.startswith(pre)})

    def silu(a):
        return a / (1 + np.exp(-a))
    t = x[0].astype(np.float64)
    logits = t @ P[pre + "gate.weight"].T.astype(np.float64)
    pr = np.exp(logits - logits.max(-1, keepdims=True))
    pr /= pr.sum(-1, keepdims=True)
    ref = np.zeros_like(t)
    for i in range(t.shape[0]):
        order = sorted(range(cfg.num_experts), key=lambda e: (-pr[i, e], e))[:cfg.num_experts_per_tok]
        for e in order:
            gw = P[pre + "experts.gate_proj.weight"][e].astype(np.float64)
            uw = P[pre + "experts.up_proj.weight"][e].astype(np.float64)
            dw = P[pre + "experts.down_proj.weight"][e].astype(np.float64)
            ref[i] += pr[i, e] * ((silu(t[i] @ gw.T) * (t[i] @ uw.T)) @ dw.T)
    sg = P[pre + "shared_expert.gate_proj.weight"].astype(np.float64)
    su = P[pre + "shared_expert.up_proj.weight"].astype(np.float64)
    sd = P[pre + "shared_expert.down_proj.weight"].astype(np.float64)
    shared = (silu(t @ sg.T) * (t @ su.T)) @ sd.T
    gate = 1 / (1 + np.exp(-(t @ P[pre + "shared_expert_gate.weight"].T.astype(np.float64))))
    ref += shared * gate
    assert np.allclose(y[0], ref, rtol=1e-4, atol=1e-5)


def test_window_mask_matches_numpy(oracle):
    import vectors
    lang = vectors.lang
    cfg = MU.gemma_config()
    model = llm.gemma3.Gemma3Model(cfg, 9)

    def f(b, v):
        (n,) = lang.unpack(b, 1, lang.shape(b, v))
        return model.window_mask(b, n, 4)
    (m,) = vectors.run(oracle, f, 1, np.zeros(9, np.float32))
    i, j = np.meshgrid(np.arange(9), np.arange(9), indexing="ij")
    masked = (j > i) | (i - j >= 4)
    assert np.array_equal(m != 0, masked)
    assert np.all(m[masked] <= np.finfo(np.float32).min)


def test_batch_folding_equals_per_sequence(oracle):
    """[B, S] ids give the same logits as running each sequence alone (batch-1, as the reference)."""
    cfg = MU.gemma_config()
    P = MU.gemma_params(cfg, seed=5, std=0.2)
    ids = np.random.default_rng(6).integers(0, cfg.vocab_size, (3, 7))
    model = llm.gemma3.Gemma3Model(cfg, 7)
    _, both = run_model(oracle, model, P, ids)
    for r in range(3):
        _, one = run_model(oracle, model, P, ids[r:r + 1])
        assert np.allclose(both[r], one[0], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["f32", "nopat", "bf16"])
def test_qwen_moe_hip_vs_oracle(oracle, hip, hip_nopat, hip_bf16, mode):
    cfg = MU.qwen_moe_config()
    P = MU.qwen_moe_params(cfg, seed=7, std=0.15)
    ids = np.random.default_rng(8).integers(0, cfg.vocab_size, (2, 9))
    model = llm.qwen_moe.QwenMoeModel(cfg, 9)
    dev = {"f32": hip, "nopat": hip_nopat, "bf16": hip_bf16}[mode]
    if mode == "bf16":
        P_ref = {k: (U_round(v) if v.ndim >= 2 else v) for k, v in P.items()}
    else:
        P_ref = P
    rt, rl = run_model(oracle, model, P_ref, ids)
    gt, gl = run_model(dev, model, P, ids)
    parity.assert_logits(rl, gl, mode, "Qwen-MoE layout")
    if mode != "bf16":
        assert np.array_equal(rt, gt)


class _QwenMoeWithRouterLogits(llm.qwen_moe.QwenMoeModel):
    """The model, with every layer's router logits ([1, B*S, E]) as extra results."""

    def sort(self):
        i, o = super().sort()
        return i, o + [o[0]] * self.config.num_hidden_layers

    def moe(self, builder, p, x):
        from importlib import import_module
        nn = import_module("catgrad-rs_amd.nn")
        c = self.config
        self._router.append(nn.linear_no_bias(builder, c.hidden_size, c.num_experts, p.extend(["gate"]), x))
        return super().moe(builder, p, x)

    def def_(self, builder, args):
        self._router = []
        out = super().def_(builder, args)
        return out + self._router


@pytest.mark.gpu
def test_qwen_moe_prefill_of_many_tokens(oracle, hip_bf16):
    """2 x 48 tokens in bf16 mode: the routed experts of a layer run expert by expert, all slots in one
    launch for gate and up and one for down_proj; same logits as the oracle on the rounded parameters."""
    cfg = MU.qwen_moe_config()
    P = MU.qwen_moe_params(cfg, seed=9, std=0.15)
    ids = np.random.default_rng(10).integers(0, cfg.vocab_size, (2, 48))
    model = llm.qwen_moe.QwenMoeModel(cfg, 48)
    P_ref = {k: (U_round(v) if v.ndim >= 2 else v) for k, v in P.items()}
    rt, rl = run_model(oracle, model, P_ref, ids)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    gt, gl = run_model(hip_bf16, model, P, ids)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    # Every token is held to the bf16 bar, except where top-k itself is discontinuous: a token whose
    # router logits - in some layer, for itself or for an earlier token of its sequence (attention
    # carries a changed token forward) - have their k-th and (k+1)-th largest closer than the bf16 bar
    # on those logits may be routed to another expert on the device than in the oracle.
    err = parity.per_row_bf16(rl, gl).reshape(ids.shape)
    outs = U.interpreter(oracle, P_ref).run(_QwenMoeWithRouterLogits(cfg, 48).term(),
                                            [oracle.tensor(np.asarray(ids, np.uint32))])
    k = cfg.num_experts_per_tok
    near_tie = np.zeros(ids.shape, bool)
    for layer in outs[2:]:
        lg = oracle.numpy(layer).reshape(ids.shape + (cfg.num_experts,)).astype(np.float64)
        srt = np.sort(lg, axis=-1)
        gap = srt[..., -k] - srt[..., -k - 1]
        near_tie |= gap <= parity.RTOL_BF16 * np.abs(lg).max(axis=-1)
    exposed = np.maximum.accumulate(near_tie, axis=1)         # the token itself or an earlier one
    over = err > parity.RTOL_BF16
    assert not (over & ~exposed).any(), (np.argwhere(over & ~exposed)[:5], err[over & ~exposed][:5])
    assert (~over).mean() >= 0.5, "most tokens must meet the bar outright"
    assert rep["gemm_experts_bf16"]["launches"] == 2 * cfg.num_hidden_layers, {k: v["launches"] for k, v in rep.items()}
    assert "gemv_experts_bf16" not in rep


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["f32", "nopat", "bf16"])
def test_gemma3_hip_vs_oracle(oracle, hip, hip_nopat, hip_bf16, mode):
    cfg = MU.gemma_config()
    P = MU.gemma_params(cfg, seed=9, std=0.2)
    ids = np.random.default_rng(10).integers(0, cfg.vocab_size, (2, 11))
    model = llm.gemma3.Gemma3Model(cfg, 11, last_position_only=True)
    dev = {"f32": hip, "nopat": hip_nopat, "bf16": hip_bf16}[mode]
    P_ref = {k: (U_round(v) if v.ndim >= 2 else v) for k, v in P.items()} if mode == "bf16" else P
    rt, rl = run_model(oracle, model, P_ref, ids)
    gt, gl = run_model(dev, model, P, ids)
    assert rl.shape == (2, 1, cfg.vocab_size)
    parity.assert_logits(rl, gl, mode, "Gemma-3")
    if mode != "bf16":
        assert np.array_equal(rt, gt)


def U_round(a):
    u = a.view(np.uint32).astype(np.uint64)
    return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("dev_name", ["hip", "hip_bf16"])
@pytest.mark.parametrize("shape", [(5, 8, 24, 64), (1, 4, 96, 1024), (33, 6, 40, 72),
                                   (200, 5, 160, 128), (1100, 3, 136, 72)])  # S, E, N, K; from 64 tokens on, bf16
                                                                              # mode multiplies expert by expert
def test_expert_indirect_matmul(request, oracle, hip_nopat, dev_name, shape):
    """matmul(x[S,1,K], transpose(1,2, index(0, idx, W[E,N,K]))) reads the expert matrices in place
    (no gather launch), with the same result as the oracle and as the gathering path."""
    import vectors
    lang = vectors.lang
    dev = request.getfixturevalue(dev_name)
    S, E, N, K = shape
    g = np.random.default_rng(S * 7 + E)
    x = g.standard_normal((S, 1, K)).astype(np.float32)
    w = g.standard_normal((E, N, K)).astype(np.float32)
    idx2 = g.integers(0, E, (S, 3)).astype(np.uint32)     # the model slices one slot of [S, k]
    if dev_name == "hip_bf16":
        w = U_round(w)

    def f(b, xv, iv, wv):
        xv = xv + xv - xv          # activations are computed values (f32), never bf16 uploads
        slot = lang.get(b, 1, 1, iv)
        sel = lang.transpose(b, 1, 2, lang.index(b, 0, slot, wv))
        return lang.matmul(b, xv, sel)
    (ref,) = vectors.run(oracle, f, 1, x, idx2, w)
    dev.trace(True)
    dev.trace_reset()
    (got,) = vectors.run(dev, f, 1, x, idx2, w)
    names = set(dev.trace_report())
    dev.trace(False)
    (gen,) = vectors.run(hip_nopat, f, 1, x, idx2, w)
    assert "gather" not in names, sorted(names)
    expect = np.einsum("sk,snk->sn", x[:, 0].astype(np.float64), w[idx2[:, 1]].astype(np.float64))
    assert np.allclose(ref[:, 0], expect, rtol=1e-4, atol=1e-3)
    tol = 2e-2 if dev_name == "hip_bf16" else 1e-4
    assert np.max(np.abs(got - ref)) <= tol * np.abs(ref).max()
    assert np.max(np.abs(gen - ref)) <= 1e-4 * np.abs(ref).max()


@pytest.mark.gpu
def test_expert_index_out_of_bounds_is_reported(hip):
    """ndarray's select panics on an index past the axis; the in-place expert read reports it."""
    import vectors
    lang = vectors.lang
    x = np.ones((2, 1, 16), np.float32)
    w = np.ones((3, 8, 16), np.float32)
    idx = np.array([1, 3], np.uint32)

    def f(b, xv, iv, wv):
        return lang.matmul(b, xv, lang.transpose(b, 1, 2, lang.index(b, 0, iv, wv)))
    with pytest.raises(cg.abi.BackendPanic, match="index out of bounds"):
        vectors.run(hip, f, 1, x, idx, w)
    # the flag is cleared: the next evaluation is clean
    (ok,) = vectors.run(hip, f, 1, x, np.array([1, 2], np.uint32), w)
    assert np.array_equal(ok, np.full((2, 1, 8), 16.0, np.float32))


@pytest.mark.gpu
def test_expert_slots_over_many_tokens(oracle, hip_bf16):
    """The routed half of the MoE block as the model emits it (models/qwen3.rs:104-123) with the indices
    given: three slots, each gate / up / SwiGLU / down over 150 tokens, weighted and summed.  All slots
    share two launches; values against the oracle."""
    import vectors
    lang, nn = vectors.lang, vectors.nn
    S, E, F, H, k = 150, 6, 64, 128, 3
    g = np.random.default_rng(6)
    x = g.standard_normal((S, 1, H)).astype(np.float32)
    wg, wu = (U_round((g.standard_normal((E, F, H)) * 0.1).astype(np.float32)) for _ in range(2))
    wd = U_round((g.standard_normal((E, H, F)) * 0.1).astype(np.float32))
    idx = g.integers(0, E, (S, k)).astype(np.uint32)
    val = g.random((S, k)).astype(np.float32)

    def f(b, xv, iv, vv, g_all, u_all, d_all):
        xv = xv + xv - xv
        total = None
        for i in range(k):
            slot = lang.get(b, 1, i, iv)
            sel = lambda w: lang.transpose(b, 1, 2, lang.index(b, 0, slot, w))
            gate = lang.matmul(b, xv, sel(g_all))
            up = lang.matmul(b, xv, sel(u_all))
            y = lang.matmul(b, nn.silu(b, gate) * up, sel(d_all))
            wgt = lang.reshape(b, lang.shape(b, lang.get(b, 2, 0, y)), lang.get(b, 1, i, vv))
            y = y * lang.broadcast(b, wgt, lang.shape(b, y))
            total = y if total is None else total + y
        return total
    (ref,) = vectors.run(oracle, f, 1, x, idx, val, wg, wu, wd)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    (got,) = vectors.run(hip_bf16, f, 1, x, idx, val, wg, wu, wd)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    assert rep["gemm_experts_bf16"]["launches"] == 2, {n: v["launches"] for n, v in rep.items()}
    assert np.max(np.abs(got - ref)) <= 2e-2 * np.abs(ref).max()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n,k", [(4, 60, 4), (7, 128, 8), (1, 256, 2), (3, 64, 64), (130, 40, 5), (2, 300, 4)])
def test_router_softmax_and_topk_in_one_launch(oracle, hip, hip_nopat, rows, n, k):
    """topk(softmax(logits)) as a MoE router emits it (models/qwen3.rs:64-80): rows of at most 256 logits
    take one launch that never stores the probabilities; same values as the two-launch path bit for bit,
    the oracle's indices, and ties (equal logits) resolved towards the lower index."""
    import vectors
    lang, nn = vectors.lang, vectors.nn
    g = np.random.default_rng(rows * n + k)
    x = (g.standard_normal((rows, 1, n)) * 3).astype(np.float32)
    x[0, 0, 5] = x[0, 0, 2] = x[0, 0].max() + 1.0          # an exact tie at the top of the first row

    def f(b, xv):
        xv = xv + xv - xv
        return lang.topk(b, k, nn.softmax(b, xv))
    rv, ri = vectors.run(oracle, f, 2, x)
    hip.trace(True)
    hip.trace_reset()
    gv, gi = vectors.run(hip, f, 2, x)
    rep = hip.trace_report()
    hip.trace(False)
    nv, ni = vectors.run(hip_nopat, f, 2, x)
    if n <= 256:
        assert "softmax_topk" in rep and "softmax_fused" not in rep and "topk" not in rep, sorted(rep)
        assert np.array_equal(gv.view(np.uint32), nv.view(np.uint32)) or np.allclose(gv, nv, rtol=1e-6, atol=0)
    else:
        assert "softmax_topk" not in rep
    assert np.array_equal(gi, ri) and np.array_equal(ni, ri)
    assert gi[0, 0, 0] == 2 and gi[0, 0, 1] == 5
    assert np.allclose(gv, rv, rtol=1e-4, atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("dev_name", ["hip", "hip_bf16"])
@pytest.mark.parametrize("S,k", [(4, 4), (1, 2), (7, 3)])
def test_expert_slots_of_a_decode_step(request, oracle, dev_name, S, k):
    """The routed half of the MoE block for the few tokens of a decode step: all k slots share one
    batched launch for gate and up and one for down_proj (with the SwiGLU in its prologue), every
    (slot, token) pair reading its expert's rows in place; an index past the last expert is reported."""
    import vectors
    lang, nn = vectors.lang, vectors.nn
    dev = request.getfixturevalue(dev_name)
    E, F, H = 6, 96, 128
    g = np.random.default_rng(S * 10 + k)
    x = g.standard_normal((S, 1, H)).astype(np.float32)
    wg, wu = ((g.standard_normal((E, F, H)) * 0.1).astype(np.float32) for _ in range(2))
    wd = (g.standard_normal((E, H, F)) * 0.1).astype(np.float32)
    if dev_name == "hip_bf16":
        wg, wu, wd = U_round(wg), U_round(wu), U_round(wd)
    idx = g.integers(0, E, (S, k)).astype(np.uint32)
    val = g.random((S, k)).astype(np.float32)

    def f(b, xv, iv, vv, g_all, u_all, d_all):
        xv = xv + xv - xv
        total = None
        for i in range(k):
            slot = lang.get(b, 1, i, iv)
            sel = lambda w: lang.transpose(b, 1, 2, lang.index(b, 0, slot, w))
            gate = lang.matmul(b, xv, sel(g_all))
            up = lang.matmul(b, xv, sel(u_all))
            y = lang.matmul(b, nn.silu(b, gate) * up, sel(d_all))
            wgt = lang.reshape(b, lang.shape(b, lang.get(b, 2, 0, y)), lang.get(b, 1, i, vv))
            y = y * lang.broadcast(b, wgt, lang.shape(b, y))
            total = y if total is None else total + y
        return total
    (ref,) = vectors.run(oracle, f, 1, x, idx, val, wg, wu, wd)
    dev.trace(True)
    dev.trace_reset()
    (got,) = vectors.run(dev, f, 1, x, idx, val, wg, wu, wd)
    rep = dev.trace_report()
    dev.trace(False)
    name = "gemv_experts_bf16" if dev_name == "hip_bf16" else "gemv_experts_f32"
    launches = {n: v["launches"] for n, v in rep.items()}
    assert launches.get(name) == 2 and "gather" not in launches and "swiglu_fused" not in launches, launches
    tol = 2e-2 if dev_name == "hip_bf16" else 1e-4
    assert np.max(np.abs(got - ref)) <= tol * np.abs(ref).max()
    bad = idx.copy()
    bad[S - 1, k - 1] = E
    with pytest.raises(cg.abi.BackendPanic, match="index out of bounds"):
        vectors.run(dev, f, 1, x, bad, val, wg, wu, wd)


@pytest.mark.gpu
@pytest.mark.parametrize("dev_name", ["hip", "hip_bf16"])
@pytest.mark.parametrize("S,E,k", [(4, 60, 4), (1, 8, 2), (7, 64, 8), (3, 5, 5)])
def test_router_choice_made_by_the_experts_launch(request, oracle, dev_name, S, E, k):
    """The same block with its router (models/qwen3.rs:64-80): slot i reads column i of topk(softmax(logits)),
    and the weights are the chosen probabilities.  With at most 64 experts the first expert launch makes the
    choice itself - no router launch - and leaves values and indices for their other readers; both must be the
    oracle's (exact ties between logits go to the lower index), whatever else reads them."""
    import vectors
    lang, nn = vectors.lang, vectors.nn
    dev = request.getfixturevalue(dev_name)
    F, H = 64, 128
    g = np.random.default_rng(S * 100 + E + k)
    x = g.standard_normal((S, 1, H)).astype(np.float32)
    logits = (g.standard_normal((1, S, E)) * 2).astype(np.float32)
    logits[0, 0, 1] = logits[0, 0, 3] = logits[0, 0].max() + 0.5        # a tie for the first choice of token 0
    wg, wu = ((g.standard_normal((E, F, H)) * 0.1).astype(np.float32) for _ in range(2))
    wd = (g.standard_normal((E, H, F)) * 0.1).astype(np.float32)
    if dev_name == "hip_bf16":   # (arrays of two or more axes are stored as bf16 in this mode: the oracle gets the same values)
        wg, wu, wd, logits = U_round(wg), U_round(wu), U_round(wd), U_round(logits)

    def f(b, xv, lv, g_all, u_all, d_all):
        xv = xv + xv - xv
        lv = lv + lv - lv
        vv, iv = lang.topk(b, k, nn.softmax(b, lv))
        sh = lang.make_shape(b, S, k)
        iv, vv = lang.reshape(b, sh, iv), lang.reshape(b, sh, vv)
        total = None
        for i in range(k):
            slot = lang.get(b, 1, i, iv)
            sel = lambda w: lang.transpose(b, 1, 2, lang.index(b, 0, slot, w))
            gate = lang.matmul(b, xv, sel(g_all))
            up = lang.matmul(b, xv, sel(u_all))
            y = lang.matmul(b, nn.silu(b, gate) * up, sel(d_all))
            wgt = lang.reshape(b, lang.shape(b, lang.get(b, 2, 0, y)), lang.get(b, 1, i, vv))
            y = y * lang.broadcast(b, wgt, lang.shape(b, y))
            total = y if total is None else total + y
        return total, iv, vv
    ref, ri, rv = vectors.run(oracle, f, 3, x, logits, wg, wu, wd)
    dev.trace(True)
    dev.trace_reset()
    got, gi, gv = vectors.run(dev, f, 3, x, logits, wg, wu, wd)
    rep = dev.trace_report()
    dev.trace(False)
    name = "gemv_experts_bf16" if dev_name == "hip_bf16" else "gemv_experts_f32"
    launches = {n: v["launches"] for n, v in rep.items()}
    assert launches.get(name) == 2 and "softmax_topk" not in launches and "topk" not in launches, launches
    assert np.array_equal(gi, ri) and ri[0, 0] == 1 and ri[0, 1] == 3
    assert np.allclose(gv, rv, rtol=1e-4, atol=1e-7)
    tol = 2e-2 if dev_name == "hip_bf16" else 1e-4
    assert np.max(np.abs(got - ref)) <= tol * np.abs(ref).max()


@pytest.mark.gpu
@pytest.mark.parametrize("norm_is_read_elsewhere", [False, True])
def test_norm_computed_by_each_reader_of_a_moe_block(oracle, hip_bf16, norm_is_read_elsewhere):
    """post-attention RMSNorm -> MoE block (qwen_moe.py `layer`) on the four rows of a decode step: when the router,
    the shared expert's gate, the shared expert's gated pair and the routed experts are the norm's only readers,
    each computes it on its way in and the norm has no launch; when anything else reads it too it is computed
    once, in memory.  The same numbers either way."""
    import vectors
    lang = vectors.lang
    cfg = MU.qwen_moe_config(num_hidden_layers=1, hidden_size=256, moe_intermediate_size=128,
                             shared_expert_intermediate_size=256)
    P = MU.qwen_moe_params(cfg, seed=31, std=0.2)
    pre = "qwen_moe.model.layers.0."
    P = {k: v for k, v in P.items() if k.startswith(pre + "mlp.") or k == pre + "post_attention_layernorm.weight"}
    P[pre + "post_attention_layernorm.weight"] = (1 + 0.1 * np.random.default_rng(5).standard_normal(cfg.hidden_size)).astype(np.float32)
    P16 = {k: (llm.random_init.bf16_round(v) if v.ndim >= 2 else v) for k, v in P.items()}
    model = llm.qwen_moe.QwenMoeModel(cfg, 8)
    x = np.random.default_rng(32).standard_normal((4, 1, cfg.hidden_size)).astype(np.float32)
    root = lang.path(["qwen_moe", "model", "layers", 0])

    def f(b, xv):
        xv = xv + xv - xv
        h = llm.helpers.rmsnorm(b, cfg.rms_norm_eps, root.extend(["post_attention_layernorm"]), xv)
        folded, bb, ss = llm.qwen_moe.fold_batch(b, h)
        y = llm.qwen_moe.unfold_batch(b, bb, ss, model.moe(b, root.extend(["mlp"]), folded)) + xv
        return [y, h] if norm_is_read_elsewhere else [y]
    n_out = 2 if norm_is_read_elsewhere else 1
    ref = vectors.run(oracle, f, n_out, x, params=P16)
    hip_bf16.launch_counts(reset=True)
    got = vectors.run(hip_bf16, f, n_out, x, params=P)
    counts = hip_bf16.launch_counts(reset=True)
    for r, a in zip(ref, got):
        assert a.shape == r.shape and np.max(np.abs(a - r)) <= 2e-2 * np.abs(r).max()
    assert counts.get("rmsnorm_fused", 0) == (1 if norm_is_read_elsewhere else 0), counts
    assert counts.get("gemv_experts_bf16") == 2 and counts.get("row_scaled_sum") == 1, counts
    # the router and the shared expert's gate ride in the launch of the shared expert's gate * up, or - when the rows
    # are in memory anyway - share a launch of their own; the router's choice is made by the first expert launch
    assert counts.get("softmax_topk", 0) == 0 and counts.get("gemv_rows_bf16") == (2 if norm_is_read_elsewhere else 1), counts


@pytest.mark.gpu
@pytest.mark.parametrize("routing", ["skewed", "two experts take every token", "1500 experts"])
def test_expert_slots_sorted_by_expert(oracle, hip_bf16, routing):
    """The same block where both products have k a multiple of 64: the (slot, token) pairs are sorted by
    expert once, cut into row tiles of 128 pairs - the launches' work list, so a crowded expert is spread over
    the device - and both launches stream their operands through LDS stages.  A skewed routing: one
    expert takes most pairs (several row tiles, the last one partly filled), one takes none, the others a few
    rows; or two experts share all pairs, five full row tiles each, and seven experts have none.  An index past
    the last expert is reported from there as well."""
    import vectors
    lang, nn = vectors.lang, vectors.nn
    S, E, F, H, k = (600 if routing == "skewed" else 640), 9, 192, 256, 2
    if routing == "1500 experts":      # more experts than the routing kernel has threads: two to a thread
        S, E, F, H = 300, 1500, 64, 64
    g = np.random.default_rng(8)
    x = g.standard_normal((S, 1, H)).astype(np.float32)
    wg, wu = (U_round((g.standard_normal((E, F, H)) * 0.1).astype(np.float32)) for _ in range(2))
    wd = U_round((g.standard_normal((E, H, F)) * 0.1).astype(np.float32))
    if routing == "skewed":
        idx = g.choice(np.array([0, 1, 2, 3, 4, 6, 7, 8]), size=(S, k), p=[.04, .04, .7, .04, .04, .04, .05, .05]).astype(np.uint32)
    elif routing == "1500 experts":
        idx = g.integers(0, E, (S, k)).astype(np.uint32)
        idx[:200, 0] = 1499             # a crowded expert at the very end: two row tiles
        idx[idx == 5] = 6
    else:
        idx = np.tile(np.array([2, 7], np.uint32), (S, 1))
    assert ((idx == 2).sum() > 3 * 128 or routing == "1500 experts") and not (idx == 5).any()
    val = g.random((S, k)).astype(np.float32)

    def f(b, xv, iv, vv, g_all, u_all, d_all):
        xv = xv + xv - xv
        total = None
        for i in range(k):
            slot = lang.get(b, 1, i, iv)
            sel = lambda w: lang.transpose(b, 1, 2, lang.index(b, 0, slot, w))
            gate = lang.matmul(b, xv, sel(g_all))
            up = lang.matmul(b, xv, sel(u_all))
            y = lang.matmul(b, nn.silu(b, gate) * up, sel(d_all))
            wgt = lang.reshape(b, lang.shape(b, lang.get(b, 2, 0, y)), lang.get(b, 1, i, vv))
            y = y * lang.broadcast(b, wgt, lang.shape(b, y))
            total = y if total is None else total + y
        return total
    (ref,) = vectors.run(oracle, f, 1, x, idx, val, wg, wu, wd)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    (got,) = vectors.run(hip_bf16, f, 1, x, idx, val, wg, wu, wd)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    launches = {n: v["launches"] for n, v in rep.items()}
    assert launches.get("gemm_experts_bf16") == 2 and launches.get("experts_route") == 1, launches
    assert np.max(np.abs(got - ref)) <= 2e-2 * np.abs(ref).max()
    # every row on its own: a token routed to the crowded expert and one routed to a quiet one
    err = np.abs(got - ref).reshape(S, -1).max(axis=1)
    assert err.max() <= 2e-2 * np.abs(ref).max()
    bad = idx.copy()
    bad[S - 1, 1] = E + 3
    with pytest.raises(cg.abi.BackendPanic, match="index out of bounds"):
        vectors.run(hip_bf16, f, 1, x, bad, val, wg, wu, wd)


@pytest.mark.gpu
def test_expert_mlp_over_many_tokens(oracle, hip_bf16):
    """One expert slot of the MoE block (models/qwen3.rs:104-123) over 300 tokens in bf16 mode: gate and
    up as expert-major products, SwiGLU computed on the way into down_proj's product; and an index
    past the last expert is reported there too."""
    import vectors
    lang, nn = vectors.lang, vectors.nn
    S, E, F, H = 300, 7, 96, 128
    g = np.random.default_rng(5)
    x = g.standard_normal((S, 1, H)).astype(np.float32)
    wg, wu = (U_round((g.standard_normal((E, F, H)) * 0.1).astype(np.float32)) for _ in range(2))
    wd = U_round((g.standard_normal((E, H, F)) * 0.1).astype(np.float32))
    idx = g.integers(0, E, (S, 1)).astype(np.uint32)

    def f(b, xv, iv, g_all, u_all, d_all):
        xv = xv + xv - xv
        sel = lambda w: lang.transpose(b, 1, 2, lang.index(b, 0, iv, w))
        gate = lang.matmul(b, xv, sel(g_all))
        up = lang.matmul(b, xv, sel(u_all))
        return lang.matmul(b, nn.silu(b, gate) * up, sel(d_all))
    (ref,) = vectors.run(oracle, f, 1, x, idx, wg, wu, wd)
    hip_bf16.trace(True)
    hip_bf16.trace_reset()
    (got,) = vectors.run(hip_bf16, f, 1, x, idx, wg, wu, wd)
    rep = hip_bf16.trace_report()
    hip_bf16.trace(False)
    assert rep["gemm_experts_bf16"]["launches"] == 2 and "gather" not in rep and "swiglu_fused" not in rep, sorted(rep)
    assert np.max(np.abs(got - ref)) <= 2e-2 * np.abs(ref).max()
    bad = idx.copy()
    bad[17, 0] = E
    with pytest.raises(cg.abi.BackendPanic, match="index out of bounds"):
        vectors.run(hip_bf16, f, 1, x, bad, wg, wu, wd)


def moe_cached_generate(be, cfg, arrays, prompts, steps):
    """Greedy tokens [steps, B] and last logits per step with the KV-cached Qwen-MoE terms."""
    r = U.CachedRunner(be, cfg, arrays, prompts.shape[1] + steps + 4,
                       prefill_cls=llm.qwen_moe.QwenMoePrefill, decode_cls=llm.qwen_moe.QwenMoeDecode)
    tok, logits = r.prefill(prompts)
    toks, lg = [], []
    for _ in range(steps):
        t = be.to_vec(tok).reshape(-1)
        toks.append(t.copy())
        lg.append(be.numpy(logits))
        tok, logits = r.step(t)
    return np.stack(toks), lg


def test_moe_cached_equals_full_recompute_on_oracle(oracle):
    """Batch of 2 prompts: the KV-cached terms give the logits of the full-recompute model."""
    cfg = MU.qwen_moe_config()
    P = MU.qwen_moe_params(cfg, seed=11, std=0.15)
    prompts = np.random.default_rng(12).integers(0, cfg.vocab_size, (2, 6))
    toks, lg = moe_cached_generate(oracle, cfg, P, prompts, 3)
    seqs = prompts.copy()
    for i in range(3):
        _, full = run_model(oracle, llm.qwen_moe.QwenMoeModel(cfg, seqs.shape[1]), P, seqs)
        assert np.allclose(lg[i][:, 0], full[:, -1], rtol=2e-4, atol=2e-5), i
        assert np.array_equal(toks[i], full[:, -1].argmax(-1))
        seqs = np.concatenate([seqs, toks[i][:, None]], axis=1)


def test_runner_generate_feeds_back_every_batch_row(oracle):
    """CachedRunner.generate / generate_pipelined with prompts [2, S]: every row's token is returned and fed
    back (the loops above are the check: they pass all rows by hand)."""
    cfg = MU.qwen_moe_config()
    P = MU.qwen_moe_params(cfg, seed=11, std=0.15)
    prompts = np.random.default_rng(12).integers(0, cfg.vocab_size, (2, 6))
    toks, _ = moe_cached_generate(oracle, cfg, P, prompts, 4)

    def runner():
        return U.CachedRunner(oracle, cfg, P, 16, prefill_cls=llm.qwen_moe.QwenMoePrefill,
                              decode_cls=llm.qwen_moe.QwenMoeDecode)
    got, _ = runner().generate(prompts, 4)
    assert got == [[int(v) for v in row] for row in toks]
    assert runner().generate_pipelined(prompts, 4) == got


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["f32", "bf16"])
def test_moe_cached_decode_hip_vs_oracle(oracle, hip, hip_bf16, mode):
    cfg = MU.qwen_moe_config()
    P = MU.qwen_moe_params(cfg, seed=13, std=0.15)
    prompts = np.random.default_rng(14).integers(0, cfg.vocab_size, (3, 9))
    dev = hip if mode == "f32" else hip_bf16
    P_ref = {k: (U_round(v) if v.ndim >= 2 else v) for k, v in P.items()} if mode == "bf16" else P
    rt, rl = moe_cached_generate(oracle, cfg, P_ref, prompts, 6)
    gt, gl = moe_cached_generate(dev, cfg, P, prompts, 6)
    compared = 0
    for i in range(6):
        parity.assert_logits(rl[i], gl[i], mode, f"step {i}")   # same history up to here
        compared += 1
        if not np.array_equal(rt[i], gt[i]):
            # the sequences part here; only on a near tie of the oracle's own top two logits may they
            # (bf16 mode), and later steps have different histories and are not comparable
            assert mode == "bf16"
            rows = np.flatnonzero(np.asarray(rt[i]).reshape(-1) != np.asarray(gt[i]).reshape(-1))
            gap = parity.top2_gap_over_max(rl[i])[rows]     # each of the two may move by the bar
            assert np.all(gap <= 2 * parity.RTOL_BF16), (i, rows, gap)
            break
    assert compared >= 1
    if mode == "f32":
        assert np.array_equal(rt, gt)


@pytest.mark.gpu
@pytest.mark.parametrize("batch,tokens,heads,kv_heads,head_dim", [(2, 256, 2, 2, 128), (1, 320, 4, 2, 128), (3, 256, 4, 4, 64),
                                                                  (4, 512, 8, 8, 128)])
def test_qwen_prefill_biases_and_rotation_in_the_projections_launch(oracle, hip_bf16, batch, tokens, heads, kv_heads, head_dim):
    """bf16 prefill of the Qwen layout (q/k/v linears with biases on the batch folded into the rows, qwen3.rs:64-133 /
    models/llama.rs:77-94): one grouped launch adds the three biases, rotates q and k and leaves the transposed bf16
    values - the trace has no bias add, rotation or transposition of its own.  Every token goes to every expert
    (k = E), so the routing has no ties to flip and the caches, the prefill's logits and a decode step's are held
    to the bf16 bar against the oracle on rounded parameters."""
    cfg = MU.qwen_moe_config(hidden_size=heads * head_dim, num_hidden_layers=2, num_attention_heads=heads,
                             num_key_value_heads=kv_heads, head_dim=head_dim, num_experts=4, num_experts_per_tok=4, vocab_size=211)
    P = MU.qwen_moe_params(cfg, seed=31, std=0.04)
    P_ref = {k: (U_round(v) if v.ndim >= 2 else v) for k, v in P.items()}
    prompts = np.random.default_rng(32).integers(0, cfg.vocab_size, (batch, tokens))
    runners = [U.CachedRunner(be, cfg, arrays, tokens + 8, prefill_cls=llm.qwen_moe.QwenMoePrefill,
                              decode_cls=llm.qwen_moe.QwenMoeDecode) for be, arrays in ((oracle, P_ref), (hip_bf16, P))]
    rt, rl = runners[0].prefill(prompts)
    hip_bf16.trace(2)
    hip_bf16.trace_reset()
    gt, gl = runners[1].prefill(prompts)
    gl = hip_bf16.numpy(gl)
    rep = hip_bf16.trace_report()
    names = sorted(rep)
    hip_bf16.trace(False)
    parity.assert_bf16(oracle.numpy(rl), gl, "prefill logits")
    assert sum("grouped,rope" in n for n in names) == 1, names
    assert not any(n.startswith(("rope_fused", "transpose_cast_bf16")) for n in names), names
    # (at most the two residual adds of a layer are launches of their own at this size; the three bias adds are not)
    assert rep.get("binary_f32", {"launches": 0})["launches"] <= 2 * cfg.num_hidden_layers, {k: v["launches"] for k, v in rep.items()}
    # The first layer's caches are that launch's own output on exact inputs: the bar.  Deeper layers see the bf16
    # rounding of a whole block first (the rounded queries and keys move the attention's scores by absolute amounts,
    # which positions with a sharp softmax amplify past the bar; f32 mode agrees to 1e-4, and the unfused kernels
    # give the same values bit for bit): there the typical position is held to it.
    for layer in range(cfg.num_hidden_layers):
        for which, what in ((0, "rotated keys"), (1, "values")):
            ref, got = oracle.numpy(runners[0].kv[2 * layer + which]), hip_bf16.numpy(runners[1].kv[2 * layer + which])
            if layer == 0:
                parity.assert_bf16(ref, got, f"layer {layer} {what}")
            else:
                assert np.median(parity.per_row_bf16(ref, got)) <= parity.RTOL_BF16, (layer, what)
    tok = oracle.to_vec(rt).reshape(-1)
    _, rl = runners[0].step(tok)
    _, gl = runners[1].step(tok)
    parity.assert_bf16(oracle.numpy(rl), hip_bf16.numpy(gl), "decode step on the prefill's caches")


@pytest.mark.gpu
def test_generic_program_launches_of_the_other_decoders(hip_bf16):
    """Which launches of a Gemma-3 prefill and of a Qwen-MoE-layout decode step are generic programs:
    the embedding scale (one per Gemma run); everything else is a pattern kernel - the weighted sum of the
    expert rows, the gated shared expert and the residual of a MoE layer are one `row_scaled_sum` launch."""
    be = hip_bf16
    gcfg = MU.gemma_config()
    P = MU.gemma_params(gcfg, seed=9, std=0.2)
    ids = np.random.default_rng(10).integers(0, gcfg.vocab_size, (2, 11)).astype(np.uint32)
    it = U.interpreter(be, P)
    term = llm.gemma3.Gemma3Model(gcfg, 11, last_position_only=True).term()
    be.to_vec(it.run(term, [be.tensor(ids)])[0])
    be.launch_counts(reset=True)
    be.to_vec(it.run(term, [be.tensor(ids)])[0])
    counts = be.launch_counts(reset=True)
    assert sum(counts.get(k, 0) for k in be.GENERIC_PROGRAMS) == 1, counts
    assert counts.get("rmsnorm_fused") == 6 * gcfg.num_hidden_layers + 1 and counts.get("geglu_fused", 0) + \
        counts.get("gemm_mfma_bf16", 0) >= gcfg.num_hidden_layers, counts
    qcfg = MU.qwen_moe_config()
    P = MU.qwen_moe_params(qcfg, seed=13, std=0.15)
    prompts = np.random.default_rng(14).integers(0, qcfg.vocab_size, (3, 9))
    r = U.CachedRunner(be, qcfg, P, 32, prefill_cls=llm.qwen_moe.QwenMoePrefill, decode_cls=llm.qwen_moe.QwenMoeDecode)
    tok, _ = r.prefill(prompts)
    t = be.to_vec(tok).reshape(-1)
    tok, _ = r.step(t)
    t = be.to_vec(tok).reshape(-1)
    be.launch_counts(reset=True)
    tok, _ = r.step(t)
    be.to_vec(tok)
    counts = be.launch_counts(reset=True)
    assert sum(counts.get(k, 0) for k in be.GENERIC_PROGRAMS) == 0, counts
    assert counts.get("row_scaled_sum") == qcfg.num_hidden_layers, counts
    # (the router's softmax and top-k are made by the routed experts' first launch, the post-attention norm by
    # each of its readers)
    assert counts.get("softmax_topk", 0) == 0 and counts.get("attn_decode") == qcfg.num_hidden_layers, counts

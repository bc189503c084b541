"""The benchmark configurations 1 (the decode launch), 2, 3 and 4 at their full shapes on the device. The whole oracle product at these sizes would take
minutes on the host, so every launch is checked on samples against the float64 dense evaluation (weights decoded by the
bit-exact unpack kernel and evaluated on the host) and through size-independent properties (linearity on integer
inputs, unit-vector read-out)."""

import numpy as np
import pytest
import torch

from _util import orc, rel_l2

pytestmark = pytest.mark.gpu

GROUP = 128
REL_L2 = 1e-3


@pytest.fixture(scope="module")
def bp():
    import deepseekternarized_amd as m

    assert torch.cuda.is_available() and m.ext() is not None
    return m


def _weights(bp, E, N, K, fmt, terms, seed):
    """Device-made weights in the bench's distribution: per term packed [E, N, Kp] and fp16 scales [E, N, G]."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    packed, scales = [], []
    for t in range(terms):
        p = torch.empty(E, N, bp.packed_cols(fmt, K), dtype=torch.uint8, device="cuda")
        for e in range(E):
            u = torch.rand(N, K, device="cuda", generator=g)
            p[e] = bp.pack(torch.where(u < 0.33, -1, torch.where(u < 0.66, 1, 0)).to(torch.int8), fmt)
        packed.append(p)
        if t == 0:
            s0 = (0.02 * torch.randn(E, N, K // GROUP, device="cuda", generator=g).abs()).half()
            scales.append(s0)
        else:
            scales.append((s0.float() * 0.25).half())
    return packed, scales


def _dense_rows(bp, packed, scales, e, rows, K, fmt):
    """float64 [len(rows), K] dequantized weight rows of expert e, summed over terms (host)."""
    idx = torch.as_tensor(rows, device="cuda")
    w = None
    for p, s in zip(packed, scales):
        t = bp.unpack(p[e][idx].contiguous(), fmt, K).cpu().numpy().astype(np.float64)
        d = t * np.repeat(s[e][idx].cpu().numpy().astype(np.float64), GROUP, axis=1)
        w = d if w is None else w + d
    return w


def test_config1_decode_gemv_full_size():
    """E = 256 experts, N = 2048, K = 7168, TQ1, one token per expert: the launch bench.py times by default, on the kernel
    chosen without a switch (rows streamed through LDS tile by tile). Sampled experts against the oracle, all rows; a
    second call adds to the first one's output (the contract: out += ...)."""
    import deepseekternarized_amd as bp
    from _util import c_gemm

    E, N, K, fmt = 256, 2048, 7168, "tq1"
    packed, scales = _weights(bp, E, N, K, fmt, 1, seed=11)
    g = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randn(E, K, device="cuda", generator=g).to(torch.bfloat16)
    offsets = torch.arange(E + 1, device="cuda", dtype=torch.int64)
    got = bp.grouped_ternary_gemm(x, None, offsets, packed, scales, K, GROUP, fmt, max_rows=1)
    assert bp.ext().last_kernel() == "fp4_tq1_t1_cw", bp.ext().last_kernel()
    assert torch.isfinite(got).all()
    xh = x.float().cpu().numpy()
    rng = np.random.default_rng(13)
    for e in sorted({0, 1, 127, 128, 254, 255, *rng.choice(E, 6, replace=False).tolist()}):
        want = np.zeros((1, N), np.float32)
        c_gemm(xh[e:e + 1], None, packed[0][e].cpu().numpy(), scales[0][e].float().cpu().numpy(), K, GROUP, fmt, out=want)
        assert rel_l2(got[e:e + 1].cpu().numpy(), want) <= REL_L2, (e, rel_l2(got[e:e + 1].cpu().numpy(), want))
    ext = bp.ext()
    twice = got.clone()
    ext.ternary_grouped_gemm(twice, x, None, offsets, packed, scales, K, GROUP, 1, None, 1)
    assert torch.equal(twice, got + got)  # (x + x is exact)


def test_config3_grouped_gemm_full_size():
    """E = 384 experts, N = 2048, K = 4096, two stacked TQ2 terms, 2048 tokens routed top-6 (12,288 rows, skewed):
    the launch bench.py times. Sampled experts x sampled output rows against float64; linearity on integer inputs."""
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.kernels.ternary_hip import gather_rows

    E, N, K, T, k, fmt = 384, 2048, 4096, 2048, 6, "tq2"
    packed, scales = _weights(bp, E, N, K, fmt, 2, seed=3)
    g = torch.Generator(device="cuda").manual_seed(4)
    logits = torch.randn(T, E, device="cuda", generator=g) * 1.5
    ids = torch.topk(torch.softmax(logits, -1), k, -1).indices.reshape(-1)
    order, offsets = bp.sort_by_expert(ids, E)
    want_order, want_offsets = orc.sort_by_expert(ids.cpu().numpy(), E)
    assert np.array_equal(order.cpu().numpy(), want_order) and np.array_equal(offsets.cpu().numpy(), want_offsets)
    x = torch.randn(T, K, device="cuda", generator=g).to(torch.bfloat16)
    xg = gather_rows(x, order, k)
    counts = np.diff(want_offsets)
    got = bp.grouped_ternary_gemm(xg, None, offsets, packed, scales, K, GROUP, fmt, max_rows=int(counts.max()))
    assert bp.ext().last_kernel().startswith("gemm_tq2"), bp.ext().last_kernel()
    assert torch.isfinite(got).all()
    rng = np.random.default_rng(5)
    # the widest, the narrowest non-empty, the first, the last and 12 random experts
    nonempty = np.flatnonzero(counts)
    pick = {int(counts.argmax()), int(nonempty[counts[nonempty].argmin()]), int(nonempty[0]), int(nonempty[-1]), *rng.choice(nonempty, 12, replace=False).tolist()}
    xg_host = xg.float().cpu().numpy().astype(np.float64)
    for e in sorted(pick):
        a, b = int(want_offsets[e]), int(want_offsets[e + 1])
        rows = np.concatenate([[0, 15, 16, N - 1], rng.choice(N, 12, replace=False)])
        want = xg_host[a:b] @ _dense_rows(bp, packed, scales, e, rows, K, fmt).T
        assert rel_l2(got[a:b][:, torch.as_tensor(rows, device="cuda")].cpu().numpy(), want) <= REL_L2, e
    # linearity on small-integer activations (every product and partial sum is exact in float32 up to the scales)
    x1 = torch.randint(-8, 9, (T * k, K), device="cuda", generator=g).to(torch.bfloat16)
    x2 = torch.randint(-8, 9, (T * k, K), device="cuda", generator=g).to(torch.bfloat16)
    f = lambda v: bp.grouped_ternary_gemm(v, None, offsets, packed, scales, K, GROUP, fmt, max_rows=int(counts.max())).double()
    lhs, rhs = f(2 * x1 - x2), 2 * f(x1) - f(x2)
    assert ((lhs - rhs).norm() / rhs.norm()).item() <= 1e-5


@pytest.mark.parametrize("T", [1, 32, 256])
def test_config2_moe_layer_full_size(T):
    """One routed-expert layer, all TQ1: hidden 4096, 64 experts, intermediate 2048, top-6 of softmax(N(0, 1.5)) logits,
    bf16 activations, through TernaryMoE; sampled tokens against oracle.moe_layer_ref (same rounding points)."""
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.moe import TernaryMoE

    H, I, E, k, fmt = 4096, 2048, 64, 6, "tq1"
    mats = {}
    for name, (n, kk), seed in (("gate", (I, H), 5), ("up", (I, H), 6), ("down", (H, I), 7)):
        p, s = _weights(bp, E, n, kk, fmt, 1, seed)
        mats[name] = (p[0], s[0])
    moe = TernaryMoE(*[[mats[n]] for n in ("gate", "up", "down")], H, I, k, fmt, GROUP, act="bf16")
    g = torch.Generator(device="cuda").manual_seed(8 + T)
    x = torch.randn(T, H, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda", generator=g) * 1.5
    got = moe(x, logits).float().cpu().numpy()
    assert got.shape == (T, H) and np.isfinite(got).all()
    sample = sorted({0, T - 1, *np.random.default_rng(T).choice(T, min(T, 3), replace=False).tolist()})
    host = {n: (mats[n][0].cpu().numpy(), mats[n][1].cpu().numpy()) for n in mats}
    experts = [tuple([(host[n][0][e], host[n][1][e])] for n in ("gate", "up", "down")) for e in range(E)]
    want = orc.moe_layer_ref(x[sample].float().cpu().numpy(), logits[sample].cpu().numpy(), experts, k, H, I, GROUP, fmt, act="bf16")
    # both sides round to bf16 at the same points; float32 summation order may flip a few roundings
    assert rel_l2(got[sample], want) <= 5e-3, rel_l2(got[sample], want)
    assert np.abs(got[sample] - want).max() <= 2e-2 * max(1.0, np.abs(want).max())


def test_config3_moe_layer_v4_full_size():
    """Config 3's layer (E = 384, H = 4096, I = 2048, two stacked TQ2 terms, 2048 tokens top-6) through the V4 engine's call
    pattern (boilerplate/engine/model.py:376-387, 407-420): sampled tokens against oracle.moe_layer_v4_ref."""
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.moe import TernaryMoE

    H, I, E, k, T, fmt = 4096, 2048, 384, 6, 2048, "tq2"
    mats = {}
    for name, (n, kk), seed in (("gate", (I, H), 3), ("up", (I, H), 4), ("down", (H, I), 5)):
        p, s = _weights(bp, E, n, kk, fmt, 2, seed)
        mats[name] = list(zip(p, s))
    moe = TernaryMoE(mats["gate"], mats["up"], mats["down"], H, I, k, fmt, GROUP, act="bf16", pattern="v4", swiglu_limit=7.0)
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(T, H, device="cuda", generator=g).to(torch.bfloat16)
    scores = torch.softmax(torch.randn(T, E, device="cuda", generator=g) * 1.5, -1)
    weights, indices = torch.topk(scores, k, -1)
    weights = weights / (weights.sum(-1, keepdim=True) + 1e-20) * 2.5  # (norm_topk_prob and route_scale, model.py:401-404)
    got = moe.routed(x, weights, indices)
    assert bp.ext().last_kernel().startswith("gemm_tq2"), bp.ext().last_kernel()
    assert got.dtype == torch.float32 and torch.isfinite(got).all()
    sample = sorted({0, T - 1, *np.random.default_rng(3).choice(T, 3, replace=False).tolist()})
    used = sorted(set(indices[sample].reshape(-1).tolist()))
    experts = [None] * E
    for e in used:
        experts[e] = tuple([(pk[e].cpu().numpy(), sc[e].cpu().numpy()) for pk, sc in mats[n]] for n in ("gate", "up", "down"))
    for e in range(E):
        if experts[e] is None:
            experts[e] = experts[used[0]]  # (never selected by the sampled tokens)
    want = orc.moe_layer_v4_ref(x[sample].float().cpu().numpy(), weights[sample].cpu().numpy(), indices[sample].cpu().numpy(), experts,
                                H, I, GROUP, fmt, act="bf16", swiglu_limit=7.0)
    gs = got[sample].cpu().numpy()
    assert rel_l2(gs, want) <= 5e-3, rel_l2(gs, want)
    assert np.abs(gs - want).max() <= 2e-2 * max(1.0, np.abs(want).max())


def test_config4_decoder_full_size():
    """The OLMoE-shaped Mode D decoder at its full shape (16 layers, hidden 2048, 16 heads, 64 experts top-8,
    intermediate 1024, vocabulary 50304, TQ2, int8 activations): a prefill and two greedy decode steps, every ternary
    linear and every MoE layer checked in place against dequantized dense torch evaluation on the same input."""
    import torch.nn.functional as F

    import deepseekternarized_amd as bp
    from deepseekternarized_amd.decoder_harness import DecoderConfig, TernaryDecoder

    cfg = DecoderConfig()
    assert (cfg.layers, cfg.hidden, cfg.heads, cfg.experts, cfg.top_k, cfg.inter, cfg.vocab, cfg.fmt, cfg.act) == \
        (16, 2048, 16, 64, 8, 1024, 50304, "tq2", "int8")
    m = TernaryDecoder(cfg, seed=1)

    def dense(packed, scale, K):
        return bp.unpack(packed, cfg.fmt, K).float() * scale.float().repeat_interleave(cfg.group, -1)[:, :K]

    def quant(x):  # boilerplate/ternary/ops.py:20-25 in torch
        xf = x.float()
        s = (xf.abs().amax(-1, keepdim=True) / 127.0).clamp(min=1e-8)
        return torch.round(xf / s).clamp(-127, 127) * s

    def lin(x, w):
        return (quant(x) @ w.t()).to(x.dtype)

    def rel(a, b):
        return ((a.float() - b.float()).norm() / b.float().norm().clamp(min=1e-6)).item()

    hip_linear, hip_moe, worst, worst_moe, checked = m.linear, m.moe, [0.0], [0.0, 0.0], [0]

    def lin32(x, w):  # the same linear without the rounding of its output to bf16
        return quant(x) @ w.t()

    def checked_linear(l, x):
        y = hip_linear(l, x)
        worst[0] = max(worst[0], rel(y, lin(x, dense(l.terms[0].packed, l.terms[0].scale, cfg.hidden))))
        checked[0] += 1
        return y

    def checked_moe(layer, z):  # boilerplate/engine/standard.py:156-176
        y = hip_moe(layer, z)
        (gp, gs), (up, us), (dp, ds) = layer.experts
        flat = z.reshape(-1, cfg.hidden)
        scores = torch.softmax(F.linear(flat, layer.router).float(), dim=-1)
        values, indices = torch.topk(scores, cfg.top_k, dim=-1)
        values = values.to(z.dtype)
        out = torch.zeros_like(flat)
        exact = torch.zeros(flat.shape, dtype=torch.float32, device=flat.device)  # the same layer with no bf16 rounding inside
        for e in range(cfg.experts):
            token, slot = torch.where(indices == e)
            if not token.numel():
                continue
            xe = flat[token]
            wg, wu, wd = dense(gp[e], gs[e], cfg.hidden), dense(up[e], us[e], cfg.hidden), dense(dp[e], ds[e], cfg.inter)
            h = F.silu(lin(xe, wg)) * lin(xe, wu)
            out.index_add_(0, token, (lin(h, wd) * values[token, slot, None]).to(out.dtype))
            h32 = F.silu(lin32(xe, wg)) * lin32(xe, wu)
            exact.index_add_(0, token, lin32(h32, wd) * values[token, slot, None].float())
        # With 8 experts per token every output passes ~12 roundings to bf16 (the reference's rounding points); which way
        # each one falls depends on the float32 summation order, so two correct evaluations differ by a few bf16 units.
        # The bar: this layer is no further from the unrounded value than the reference-order torch evaluation is.
        worst_moe[0] = max(worst_moe[0], rel(y, exact.view(z.shape)) / max(rel(out.view(z.shape), exact.view(z.shape)), 1e-6))
        worst_moe[1] = max(worst_moe[1], rel(y, out.view(z.shape)))
        checked[0] += 1
        return y

    m.linear, m.moe = checked_linear, checked_moe
    ids = torch.randint(0, cfg.vocab, (4, 16), generator=torch.Generator().manual_seed(2))
    logits, cache = m.forward(ids)
    assert logits.shape == (4, 16, cfg.vocab) and torch.isfinite(logits).all()
    nxt = logits[:, -1].argmax(-1)
    for _ in range(2):
        logits, cache = m.forward(nxt[:, None].cpu(), cache)
        assert torch.isfinite(logits).all()
        nxt = logits[:, -1].argmax(-1)
    assert checked[0] == 3 * cfg.layers * 3  # per forward and layer: q|k|v (one stacked linear), o, the MoE
    assert worst[0] <= 5e-3, worst[0]  # single linears, bf16 outputs: a few roundings flip on float32 summation order
    assert worst_moe[0] <= 1.25 and worst_moe[1] <= 1.5e-2, worst_moe


def test_config4_decode_step_at_the_benchmark_batch():
    """The decode step `bench.py` times (64 sequences, 128-token prompt): one eager step with every ternary linear
    checked in place against dequantized dense torch evaluation on sampled rows, and the same step replayed as a HIP
    graph against the eager logits."""
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.decoder_harness import DecoderConfig, GraphedDecode, TernaryDecoder

    cfg = DecoderConfig()
    m = TernaryDecoder(cfg, seed=5)

    def dense(packed, scale, K):
        return bp.unpack(packed, cfg.fmt, K).float() * scale.float().repeat_interleave(cfg.group, -1)[:, :K]

    def quant(x):  # boilerplate/ternary/ops.py:20-25 in torch
        xf = x.float()
        s = (xf.abs().amax(-1, keepdim=True) / 127.0).clamp(min=1e-8)
        return torch.round(xf / s).clamp(-127, 127) * s

    hip_linear, worst, checked, on = m.linear, [0.0], [0], [False]

    def checked_linear(l, x):
        y = hip_linear(l, x)
        if on[0]:
            flat, yf = x.reshape(-1, x.shape[-1])[::7], y.reshape(-1, y.shape[-1])[::7]
            want = (quant(flat) @ dense(l.terms[0].packed, l.terms[0].scale, cfg.hidden).t()).to(y.dtype)
            worst[0] = max(worst[0], ((yf.float() - want.float()).norm() / want.float().norm().clamp(min=1e-6)).item())
            checked[0] += 1
        return y

    m.linear = checked_linear
    ids = torch.randint(0, cfg.vocab, (64, 128), generator=torch.Generator().manual_seed(6))
    logits, cache = m.forward(ids)
    assert torch.isfinite(logits[:, -1]).all()
    nxt = logits[:, -1].argmax(-1)
    del logits
    dec = GraphedDecode(m, cache, max_len=128 + 4)
    on[0] = True
    want, cache = m.forward(nxt[:, None].cpu(), cache)
    on[0] = False
    torch.cuda.synchronize()
    assert checked[0] == 2 * cfg.layers and worst[0] <= 5e-3, (checked[0], worst[0])
    got = dec.step(nxt).clone()
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    rel = ((got.float() - want[:, 0].float()).norm() / want[:, 0].float().norm()).item()
    assert rel <= 2e-2, rel
    assert (got.argmax(-1) == want[:, 0].argmax(-1)).float().mean().item() >= 0.9

"""bp_moe_layer_bf16 (one library call per MoE layer, no host synchronisation, caller's workspace) against the same layer
composed of separate library calls with the reference's host-side sizing (boilerplate/kernels/ternary_cuda.py:97), and
against the CPU restatement of boilerplate/engine/standard.py:151-176 (oracle.moe_layer_ref)."""

import ctypes as C

import numpy as np
import pytest
import torch

from oracle import ternary_oracle as orc

pytestmark = pytest.mark.gpu


def _layer(fmt, act, H, I, E, k, terms=1, seed=0, sdtype=torch.float16):
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.moe import TernaryMoE

    g = torch.Generator(device="cuda").manual_seed(seed)
    mats = []
    for n, kk in ((I, H), (I, H), (H, I)):
        ts = []
        for t in range(terms):
            u = torch.rand(E, n, kk, device="cuda", generator=g)
            tr = torch.where(u < 0.3, -1, torch.where(u < 0.6, 1, 0)).to(torch.int8)
            pk = torch.stack([bp.pack(tr[e], fmt) for e in range(E)])
            sc = (0.04 * torch.randn(E, n, kk // 128, device="cuda", generator=g).abs() * 0.25 ** t).to(sdtype)
            ts.append((pk, sc))
        mats.append(ts)
    return TernaryMoE(*mats, H, I, k, fmt, 128, act=act), mats


def _rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm().clamp(min=1e-9)).item()


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("T", [1, 7, 64])
def test_layer_call_equals_composed_calls_up_to_64_tokens(fmt, act, T):
    """Up to 64 tokens both paths size the grouped launches by the same bound: the same kernels, bit-identical outputs."""
    moe, _ = _layer(fmt, act, 1024, 1024, 8, 2, seed=T)
    g = torch.Generator(device="cuda").manual_seed(100 + T)
    x = torch.randn(T, 1024, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, 8, device="cuda", generator=g)
    got, want = moe(x, logits), moe.composed(x, logits)
    assert got.shape == want.shape == (T, 1024) and torch.isfinite(got.float()).all()
    assert torch.equal(got, want)


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("fmt,terms", [("tq1", 1), ("tq2", 2)])
def test_layer_call_over_the_tile_list_matches_composed_calls(fmt, terms, act):
    """Beyond 64 tokens the call runs the grouped GEMMs over the device-side tile list. Skewed routing: an expert with no
    row, experts with 1..31 rows, one with several tiles and a ragged last tile."""
    from deepseekternarized_amd import ext

    H, I, E, k, T = 1024, 2048, 16, 2, 300
    moe, _ = _layer(fmt, act, H, I, E, k, terms=terms, seed=3)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(T, H, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda", generator=g)
    logits[:, 0] += 4.0    # nearly every token routes to expert 0: 300 rows = 10 tiles, the last one ragged
    logits[:, 9] = -40.0   # expert 9 gets nothing
    logits[:, 11] -= 2.5   # a handful of rows
    got = moe(x, logits)
    assert ext().last_kernel().startswith("gemm_" + fmt), ext().last_kernel()
    want = moe.composed(x, logits)
    assert torch.isfinite(got.float()).all()
    # the composed path may pick other kernels for the same rows (its bound is exact): same rounding points, float32 sums in another order
    assert _rel(got, want) <= 2e-3, _rel(got, want)
    # the same call again: identical (nothing of the previous call is left in the workspace that matters)
    assert torch.equal(moe(x, logits), got)
    # fewer tokens through the same (larger) workspace
    got2 = moe(x[:70], logits[:70])
    assert _rel(got2, moe.composed(x[:70], logits[:70])) <= 2e-3


def test_layer_call_over_the_tile_list_with_converted_activations(tune):
    """TQ2, bf16 activations, beyond 64 tokens: the workspace has room for the activations converted to fp8 pieces, and the
    grouped GEMMs over them read the same device-side tile list (forced here: the shape is below that kernel's thresholds)."""
    from deepseekternarized_amd import ext

    H, I, E, k, T = 1024, 2048, 16, 2, 300
    moe, _ = _layer("tq2", "bf16", H, I, E, k, terms=2, seed=3)
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(T, H, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda", generator=g)
    logits[:, 0] += 4.0
    logits[:, 9] = -40.0
    logits[:, 11] -= 2.5
    tune("BP_TUNE_TQ2G", "fp4")
    got = moe(x, logits).clone()
    assert ext().last_kernel() == "gemm_tq2f_bf16+glu+gather+y16", ext().last_kernel()  # (the gate | up launch gathered its rows and applied SwiGLU itself)
    assert torch.equal(moe(x, logits), got)
    tune("BP_TUNE_TQ2G", "bf16")
    want = moe(x, logits)
    assert ext().last_kernel().startswith("gemm_tq2_bf16"), ext().last_kernel()
    assert torch.isfinite(got.float()).all() and _rel(got, want) <= 2e-3, _rel(got, want)


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_layer_call_matches_the_reference_loop(fmt, act):
    """Against the per-expert loop of boilerplate/engine/standard.py:151-176 restated on the CPU, 96 tokens (tile-list path)."""
    H, I, E, k, T, group = 1024, 1024, 8, 2, 96, 128
    moe, mats = _layer(fmt, act, H, I, E, k, seed=11)
    rng = np.random.default_rng(12)
    x = orc.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    logits = (rng.standard_normal((T, E)) * 1.5).astype(np.float32)
    logits[:, 5] = -30.0
    experts = [tuple([(mats[n][0][0][e].cpu().numpy(), mats[n][0][1][e].cpu().numpy())] for n in range(3)) for e in range(E)]
    want = orc.moe_layer_ref(x, logits, experts, k, H, I, group, fmt, act=act)
    got = moe(torch.from_numpy(x).cuda().to(torch.bfloat16), torch.from_numpy(logits).cuda()).float().cpu().numpy()
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel <= 5e-3, rel  # bf16 at the same points; float32 summation order flips a few roundings


def test_layer_call_as_a_graph_beyond_64_tokens():
    """No read-back anywhere: 128 tokens captured as one HIP graph, replayed with eager work in between."""
    moe, _ = _layer("tq2", "bf16", 1024, 1024, 8, 2, seed=21)
    run = moe.graphed(128)
    g = torch.Generator(device="cuda").manual_seed(22)
    for rep in range(3):
        x = torch.randn(128, 1024, device="cuda", generator=g).to(torch.bfloat16)
        logits = torch.randn(128, 8, device="cuda", generator=g)
        want = moe(x, logits).clone()
        torch.cuda.synchronize()
        got = run(x, logits).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


def test_layer_call_argument_checks():
    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    moe, _ = _layer("tq2", "bf16", 1024, 1024, 8, 2, seed=31)
    T = 4
    x = torch.zeros(T, 1024, dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(x)
    idx = torch.zeros(T, 2, dtype=torch.int64, device="cuda")
    idx[:, 1] = 1
    w = torch.ones(T, 2, dtype=torch.bfloat16, device="cuda")
    need = lib.bp_moe_layer_workspace_bytes(T, 1024, 1024, 8, 2, _lib.BP_BF16, 2)
    assert need > 0 and need % 256 == 0
    assert lib.bp_moe_layer_workspace_bytes(T, 1024, 1024, 8, 2, _lib.BP_I8, 2) not in (0, need)  # (int8: the quantized rows and their scales instead of converted activations)
    # bf16 activations: room for the converted activations of a grouped GEMM as well (both formats)
    assert lib.bp_moe_layer_workspace_bytes(128, 1024, 1024, 8, 2, _lib.BP_BF16, 2) == lib.bp_moe_layer_workspace_bytes(128, 1024, 1024, 8, 2, _lib.BP_BF16, 1)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    arr = lambda ts: (C.c_void_p * 1)(*[t.data_ptr() for t in ts])
    gp, gs = arr([moe.gate_up[0][0]]), arr([moe.gate_up[0][1]])
    dp, ds = arr([moe.down[0][0]]), arr([moe.down[0][1]])

    def call(**kw):
        a = dict(out=out.data_ptr(), x=x.data_ptr(), idx=idx.data_ptr(), w=w.data_ptr(), T=T, H=1024, I=1024, E=8, k=2, fmt=2,
                 act=_lib.BP_BF16, ws=ws.data_ptr(), ws_bytes=need)
        a.update(kw)
        return lib.bp_moe_layer_bf16(a["out"], a["x"], a["idx"], a["w"], gp, gs, dp, ds, _lib.BP_F16, 1, a["T"], a["H"], a["I"], a["E"],
                                     a["k"], 128, a["fmt"], a["act"], a["ws"], a["ws_bytes"], None, None)

    assert call() == 0
    torch.cuda.synchronize()
    for bad in (dict(ws_bytes=need - 1), dict(ws=None), dict(ws=ws.data_ptr() + 8), dict(k=0), dict(k=9), dict(fmt=3), dict(act=_lib.BP_F32),
                dict(H=1020), dict(x=None), dict(E=70000)):
        assert call(**bad) != 0, bad
        assert lib.bp_last_error()
    assert call(T=0) == 0
    # an expert id out of range raises the flag and faults nothing
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    idx2 = idx.clone()
    idx2[1, 1] = 99
    rc = lib.bp_moe_layer_bf16(out.data_ptr(), x.data_ptr(), idx2.data_ptr(), w.data_ptr(), gp, gs, dp, ds, _lib.BP_F16, 1, T, 1024, 1024, 8, 2,
                               128, 2, _lib.BP_BF16, ws.data_ptr(), need, flag.data_ptr(), None)
    torch.cuda.synchronize()
    assert rc == 0 and int(flag) == 1


# --------------------------------------------------------------------------- the V4 engine's call pattern
def _v4_inputs(T, H, E, k, seed):
    rng = np.random.default_rng(seed)
    x = orc.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    scores = orc.softmax_f32((rng.standard_normal((T, E)) * 1.5).astype(np.float32))
    _, indices = orc.topk_desc(scores, k)
    weights = (np.take_along_axis(scores, indices, -1) * np.float32(2.5)).astype(np.float32)
    return x, weights, indices


@pytest.mark.parametrize("limit", [0.0, 0.5])
@pytest.mark.parametrize("fmt,terms,act,T", [("tq1", 1, "bf16", 96), ("tq2", 2, "bf16", 96), ("tq2", 1, "int8", 40), ("tq1", 1, "int8", 5)])
def test_v4_layer_matches_the_reference_lines(fmt, terms, act, T, limit):
    """bp_moe_layer_v4 against boilerplate/engine/model.py:376-387 / :407-420 restated on the CPU (oracle.moe_layer_v4_ref):
    float32 routing weights before w2, the clamps, float32 accumulation over a token's experts."""
    from deepseekternarized_amd.moe import TernaryMoE

    H, I, E, k, group = 1024, 1024, 8, 2, 128
    _, mats = _layer(fmt, act, H, I, E, k, terms=terms, seed=41)
    moe = TernaryMoE(*mats, H, I, k, fmt, group, act=act, pattern="v4", swiglu_limit=limit)
    x, weights, indices = _v4_inputs(T, H, E, k, seed=42 + T)
    experts = [tuple([(mats[n][t][0][e].cpu().numpy(), mats[n][t][1][e].cpu().numpy()) for t in range(terms)] for n in range(3)) for e in range(E)]
    want = orc.moe_layer_v4_ref(x, weights, indices, experts, H, I, group, fmt, act=act, swiglu_limit=limit)
    xd = torch.from_numpy(x).cuda().to(torch.bfloat16)
    got = moe.routed(xd, torch.from_numpy(weights).cuda(), torch.from_numpy(indices).cuda())
    assert got.dtype == torch.float32 and got.shape == (T, H)
    rel = np.linalg.norm(got.cpu().numpy() - want) / np.linalg.norm(want)
    assert rel <= 5e-3, rel  # the same rounding points; float32 sums in another order flip a few bf16 roundings
    # the bf16 form is the float32 one cast once
    got16 = moe.routed(xd, torch.from_numpy(weights).cuda(), torch.from_numpy(indices).cuda(), out_dtype=torch.bfloat16)
    assert torch.equal(got16, got.to(torch.bfloat16))
    if limit > 0:  # the clamp changes the result (it is exercised), and a different pattern is a different number
        free = TernaryMoE(*mats, H, I, k, fmt, group, act=act, pattern="v4").routed(xd, torch.from_numpy(weights).cuda(), torch.from_numpy(indices).cuda())
        assert not torch.equal(free, got)
    with pytest.raises(RuntimeError):
        moe(xd, torch.zeros(T, E, device="cuda"))


@pytest.mark.parametrize("pattern,limit", [("standard", 0.0), ("v4", 0.0), ("v4", 0.75)])
@pytest.mark.parametrize("fmt,terms,I", [("tq1", 1, 1024), ("tq2", 2, 1280), ("tq1", 2, 768 + 512)])
def test_swiglu_in_the_gate_up_epilogue_equals_the_separate_launch(tune, fmt, terms, I, pattern, limit):
    """Over the tile list with converted activations the gate | up launch reads its rows through the sort order (no routed
    copy of the activations), applies SwiGLU to its own float32 sums and writes bf16 h (boilerplate/engine/standard.py:151-176, boilerplate/engine/model.py:376-387): the same sums, the same
    rounding points - bit-identical to the layer with the separate SwiGLU launch (BP_TUNE_GLU=n), for both call patterns.
    Skewed routing: an expert without rows, ragged last tiles, tiles of at most 16 rows."""
    from deepseekternarized_amd import ext
    from deepseekternarized_amd.moe import TernaryMoE

    H, E, k, T = 1024, 16, 2, 200
    _, mats = _layer(fmt, "bf16", H, I, E, k, terms=terms, seed=I + terms)
    moe = TernaryMoE(*mats, H, I, k, fmt, 128, act="bf16", pattern=pattern, **({"swiglu_limit": limit} if pattern == "v4" else {}))
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.randn(T, H, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda", generator=g)
    logits[:, 0] += 4.0
    logits[:, 9] = -40.0
    logits[:, 11] -= 2.5
    if pattern == "v4":
        scores = torch.softmax(logits.float(), -1)
        w, idx = torch.topk(scores, k, dim=-1)
        run = lambda: moe.routed(x, w * 2.5, idx).clone()
    else:
        run = lambda: moe(x, logits).clone()
    if fmt == "tq2":
        tune("BP_TUNE_TQ2G", "fp4")  # (the shape is below the thresholds of the kernel over converted activations)
    fused = run()
    assert ext().last_kernel() == "gemm_%sf_bf16+glu+gather+y16" % fmt, ext().last_kernel()
    tune("BP_TUNE_GLU", "g")  # the routed copy of the activations written by a launch of its own
    assert torch.equal(run(), fused)
    assert ext().last_kernel() == "gemm_%sf_bf16+glu+y16" % fmt, ext().last_kernel()
    tune("BP_TUNE_GLU", "n")
    apart = run()
    assert ext().last_kernel() == "gemm_%sf_bf16" % fmt, ext().last_kernel()
    assert torch.isfinite(fused.float()).all() and torch.equal(fused, apart)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_swiglu_epilogue_with_a_partly_filled_row_block(tune, fmt):
    """An intermediate size that is not a multiple of the 256 rows a row block takes of either half (1152 = 4.5 blocks): the
    last block's waves without rows store nothing, and the down projection (K = 1152 is outside the tile kernels) runs
    on another kernel from the same bf16 h. Bit-identical to the separate SwiGLU launch."""
    from deepseekternarized_amd import ext

    H, I, E, k, T = 1024, 1152, 8, 2, 150
    moe, _ = _layer(fmt, "bf16", H, I, E, k, terms=1, seed=77)
    g = torch.Generator(device="cuda").manual_seed(78)
    x = torch.randn(T, H, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda", generator=g)
    if fmt == "tq2":
        tune("BP_TUNE_TQ2G", "fp4")
    fused = moe(x, logits).clone()
    assert "+glu" in ext().last_kernel(), ext().last_kernel()
    tune("BP_TUNE_GLU", "n")
    apart = moe(x, logits).clone()
    assert "+glu" not in ext().last_kernel(), ext().last_kernel()
    assert torch.isfinite(fused.float()).all() and torch.equal(fused, apart)
    assert _rel(fused, moe.composed(x, logits)) <= 2e-3


def test_v4_stages_bit_exact():
    """bp_swiglu_v4 and bp_moe_combine_v4 alone, against their definitions evaluated with torch on the device
    (float32 throughout; expf may differ from torch's by an ulp, which the bf16 rounding rarely sees)."""
    import torch.nn.functional as F

    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    g = torch.Generator(device="cuda").manual_seed(7)
    rows, I, pairs = 37, 520, 37
    gu = torch.randn(rows, 2 * I, device="cuda", generator=g) * 2
    w = torch.rand(pairs, device="cuda", generator=g) * 3
    order = torch.randperm(pairs, device="cuda", generator=g)
    h = torch.empty(rows, I, dtype=torch.bfloat16, device="cuda")
    for limit in (0.0, 1.25):
        rc = lib.bp_swiglu_v4(h.data_ptr(), gu.data_ptr(), gu[:, I:].data_ptr(), w.data_ptr(), order.data_ptr(), pairs, limit, rows, I, 2 * I, None)
        assert rc == 0, lib.bp_last_error()
        gate, up = gu[:, :I].to(torch.bfloat16).float(), gu[:, I:].to(torch.bfloat16).float()
        if limit > 0:
            up, gate = torch.clamp(up, min=-limit, max=limit), torch.clamp(gate, max=limit)
        want = (w[order][:, None] * (F.silu(gate) * up)).to(torch.bfloat16)
        same = (h == want).float().mean().item()
        assert same >= 0.999, same
        assert ((h.float() - want.float()).abs() <= want.float().abs() * 2.0 ** -7 + 1e-30).all()
    # no weights: a shared expert
    rc = lib.bp_swiglu_v4(h.data_ptr(), gu.data_ptr(), gu[:, I:].data_ptr(), None, None, 0, 0.0, rows, I, 2 * I, None)
    assert rc == 0
    want = (F.silu(gu[:, :I].to(torch.bfloat16).float()) * gu[:, I:].to(torch.bfloat16).float()).to(torch.bfloat16)
    assert (h == want).float().mean().item() >= 0.999
    # combine: float32 sums in ascending expert order of the bf16-rounded rows
    T, k, H = 9, 4, 300
    experts = torch.stack([torch.randperm(16, device="cuda", generator=g)[:k] for _ in range(T)])
    flat_order = torch.argsort(experts.reshape(-1), stable=True)
    inv = torch.empty_like(flat_order)
    inv[flat_order] = torch.arange(T * k, device="cuda")
    y = torch.randn(T * k, H, device="cuda", generator=g) * 100
    out = torch.empty(T, H, device="cuda")
    assert lib.bp_moe_combine_v4(out.data_ptr(), _lib.BP_F32, y.data_ptr(), inv.data_ptr(), experts.data_ptr(), T, k, H, None) == 0
    want = torch.zeros(T, H, device="cuda")
    yb = y.to(torch.bfloat16).float()
    for e in range(16):
        tok, slot = torch.where(experts == e)
        if tok.numel():
            want[tok] += yb[inv[tok * k + slot]]
    assert torch.equal(out, want)
    assert lib.bp_moe_combine_v4(out.data_ptr(), _lib.BP_I8, y.data_ptr(), inv.data_ptr(), experts.data_ptr(), T, k, H, None) != 0


def test_graphs_of_one_layer_keep_their_workspaces():
    """Two graphed callables of one layer and a larger eager call in between: every graph replays into the workspace it
    captured, which the layer keeps alive when a later call needs a bigger one."""
    moe, _ = _layer("tq2", "bf16", 1024, 1024, 8, 2, seed=51)
    g = torch.Generator(device="cuda").manual_seed(52)
    g1 = moe.graphed(8)
    g2 = moe.graphed(40)
    x300 = torch.randn(300, 1024, device="cuda", generator=g).to(torch.bfloat16)
    l300 = torch.randn(300, 8, device="cuda", generator=g)
    big = moe(x300, l300).clone()
    filler = [torch.randn(1 << 20, device="cuda") for _ in range(8)]  # takes freed blocks, if any were freed
    for run, T in ((g1, 8), (g2, 40), (g1, 8)):
        x = torch.randn(T, 1024, device="cuda", generator=g).to(torch.bfloat16)
        lg = torch.randn(T, 8, device="cuda", generator=g)
        want = moe(x, lg).clone()
        got = run(x, lg).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), T
    assert torch.equal(moe(x300, l300), big)
    del filler


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,renorm", [(1, 64, 6, False), (37, 64, 8, True), (300, 384, 6, False), (5, 1024, 16, True), (9, 7, 7, False), (4, 130, 1, True)])
def test_router_softmax_and_topk_in_one_launch(T, E, k, renorm, dtype):
    """bp_route_topk against the oracle's float32 softmax and stable top-k (boilerplate/engine/standard.py:160-165) and
    against torch's own ops on the device: the same experts in the same slots wherever the scores involved are further
    apart than float32 rounding, weights equal to within one bf16 step."""
    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    g = torch.Generator(device="cuda").manual_seed(T * 1000 + E)
    logits = (torch.randn(T, E, device="cuda", generator=g) * 1.5).to(dtype)
    for wdt, code in ((torch.bfloat16, _lib.BP_BF16), (torch.float32, _lib.BP_F32)):
        w = torch.full((T, k), -1.0, dtype=wdt, device="cuda")
        ids = torch.full((T, k), -1, dtype=torch.int64, device="cuda")
        _lib.check(lib.bp_route_topk(w.data_ptr(), code, ids.data_ptr(), logits.data_ptr(), _lib.dtype_code(dtype), T, E, k, int(renorm),
                                     _lib.stream_ptr(logits.device)))
        torch.cuda.synchronize()
        scores = orc.softmax_f32(logits.float().cpu().numpy())
        want_v, want_i = orc.topk_desc(scores, k)
        srt = -np.sort(-scores, axis=-1)
        # tokens whose k + 1 largest scores are equal (equal logits: the lower expert wins, here as in the oracle) or
        # further apart than the rounding of a float32 softmax; `strict`: no equal ones either (torch.topk's choice
        # among equal scores is its own)
        gaps = np.abs(np.diff(srt[:, : min(k + 1, E)], axis=-1))
        clear = ((gaps == 0) | (gaps > 4e-6 * srt[:, :1])).all(-1)
        strict = (gaps > 4e-6 * srt[:, :1]).all(-1)
        assert clear.mean() > 0.5
        got_i = ids.cpu().numpy()
        assert np.array_equal(got_i[clear], want_i[clear])
        assert ((got_i >= 0) & (got_i < E)).all() and all(len(set(r)) == k for r in got_i.tolist())
        if renorm:
            want_v = want_v / want_v.sum(-1, keepdims=True, dtype=np.float32)
        got_v = w.float().cpu().numpy()
        tol = 2.0 ** -8 if wdt == torch.bfloat16 else 2e-6
        assert np.all(np.abs(got_v[clear] - want_v[clear]) <= tol * np.abs(want_v[clear]) + 1e-30)
        # torch on the device, as the reference computes it
        tv, ti = torch.topk(torch.softmax(logits.float(), -1), k, dim=-1)
        assert np.array_equal(ti.cpu().numpy()[strict], got_i[strict])


def test_router_kernel_ties_go_to_the_lower_expert_and_bad_arguments_are_rejected():
    from deepseekternarized_amd.kernels import _lib

    lib = _lib.load()
    logits = torch.zeros(3, 200, device="cuda")
    logits[1, 150] = logits[1, 20] = 2.0  # two equal maxima, then all the zeros
    w = torch.empty(3, 4, device="cuda")
    ids = torch.empty(3, 4, dtype=torch.int64, device="cuda")
    _lib.check(lib.bp_route_topk(w.data_ptr(), _lib.BP_F32, ids.data_ptr(), logits.data_ptr(), _lib.BP_F32, 3, 200, 4, 0, _lib.stream_ptr(logits.device)))
    torch.cuda.synchronize()
    assert ids.cpu().tolist() == [[0, 1, 2, 3], [20, 150, 0, 1], [0, 1, 2, 3]]
    assert torch.allclose(w[0].cpu(), torch.full((4,), 1 / 200))
    assert lib.bp_route_topk(w.data_ptr(), _lib.BP_F32, ids.data_ptr(), logits.data_ptr(), _lib.BP_F32, 3, 2000, 4, 0, None) == 1
    assert b"1024 experts" in lib.bp_last_error()
    assert lib.bp_route_topk(w.data_ptr(), _lib.BP_I8, ids.data_ptr(), logits.data_ptr(), _lib.BP_F32, 3, 200, 4, 0, None) == 1
    assert lib.bp_route_topk(w.data_ptr(), _lib.BP_F32, ids.data_ptr(), logits.data_ptr(), _lib.BP_F32, 3, 3, 4, 0, None) == 1


@pytest.mark.parametrize("T,E,k", [(25, 8, 2), (40, 4, 2), (42, 16, 6), (33, 3, 3)])
def test_small_batch_preparation_kernel_writes_the_tile_list(T, E, k):
    """Between 24 tokens (TQ1, bf16: the tile list takes over) and 256 routed rows the preparation kernel also writes the
    list of token tiles - experts without rows, experts with more than one tile of 32 rows - and the layer equals the
    composed calls bit for bit (the same GEMM kernel, sized by the bound instead of the list)."""
    from deepseekternarized_amd import ext

    moe, _ = _layer("tq1", "bf16", 1024, 1024, E, k, seed=T)
    g = torch.Generator(device="cuda").manual_seed(7 * T)
    x = torch.randn(T, 1024, device="cuda", generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device="cuda", generator=g) * 2.0
    logits[:, 0] -= 30.0  # expert 0 gets no row
    if E == 4:
        logits[:, 1] += 6.0  # expert 1 is in every token's top-2: more than one tile
    got = moe(x, logits)
    assert ext().last_kernel() == "gemm_tq1f_bf16+glu+gather+y16", ext().last_kernel()
    want = moe.composed(x, logits)
    assert torch.isfinite(got.float()).all() and torch.equal(got, want)

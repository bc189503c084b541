"""Pins the NumPy oracle (oracle/ternary_oracle.py) without the reference: literal byte vectors
worked out by hand from the format definition, exhaustive enumeration, a digit-by-digit brute
force, closed-form special cases and the invariants the reference's own tests state
(reference tests/test_ternary.py:14-29,78-82; tests/test_ternary_cuda.py:21-57)."""

import itertools

import numpy as np
import pytest

from _util import orc


# ---- literal vectors: byte = u0 | u1<<2 | u2<<4 | u3<<6 ; byte = u0 + 3u1 + 9u2 + 27u3 + 81u4 ; u = t + 1
def test_tq2_literal_bytes():
    t = np.array([[-1, 0, 1, 1, -1]], dtype=np.int8)  # digits 0 1 2 2 | 0 + pads 1 1 1
    assert orc.pack(t, "tq2").tolist() == [[0 | 1 << 2 | 2 << 4 | 2 << 6, 0 | 1 << 2 | 1 << 4 | 1 << 6]] == [[164, 84]]
    assert orc.unpack(np.array([[164, 84]], np.uint8), "tq2", 5).tolist() == t.tolist()
    # the never-produced code 3 decodes to +2 (pack.py:9, unpack: ((b >> s) & 3) - 1)
    assert orc.unpack(np.array([[0b11100100]], np.uint8), "tq2", 4).tolist() == [[-1, 0, 1, 2]]


def test_tq1_literal_bytes():
    t = np.array([[-1, 0, 1, 1, -1, 1, 0]], dtype=np.int8)  # digits 0 1 2 2 0 | 2 1 + pads 1 1 1
    assert orc.pack(t, "tq1").tolist() == [[0 + 3 + 18 + 54 + 0, 2 + 3 + 9 + 27 + 81]] == [[75, 122]]
    assert orc.unpack(np.array([[75, 122]], np.uint8), "tq1", 7).tolist() == t.tolist()
    lut = orc.tq1_lut()
    assert lut.shape == (256, 5) and lut.dtype == np.int8
    assert lut[0].tolist() == [-1] * 5 and lut[242].tolist() == [1] * 5 and lut[121].tolist() == [0] * 5
    assert lut[1].tolist() == [0, -1, -1, -1, -1] and lut[81].tolist() == [-1, -1, -1, -1, 0]
    assert not lut[243:].any()  # rows >= 243 decode as 0


@pytest.mark.parametrize("fmt", ["tq2", "tq1"])
@pytest.mark.parametrize("K", [1, 4, 5, 7, 128, 131, 640])
def test_pack_roundtrip(fmt, K):
    rng = np.random.default_rng(K)
    t = rng.integers(-1, 2, (9, K)).astype(np.int8)
    p = orc.pack(t, fmt)
    assert p.dtype == np.uint8 and p.shape == (9, orc.packed_cols(fmt, K))
    assert np.array_equal(orc.unpack(p, fmt, K), t)


def test_tq1_every_byte_pattern():
    pats = np.array(list(itertools.product([-1, 0, 1], repeat=5)), dtype=np.int8)
    p = orc.pack(pats, "tq1")
    assert np.unique(p).size == 243 and int(p.max()) < 243
    assert np.array_equal(orc.unpack(p, "tq1", 5), pats)
    assert orc.bits_per_weight("tq1") == 1.6 and orc.bits_per_weight("tq2") == 2.0


@pytest.mark.parametrize("fmt,per", [("tq2", 4), ("tq1", 5)])
def test_pack_matches_bruteforce_digits(fmt, per):
    """Pure-Python restatement from the prose definition, one digit at a time, incl. the padding rule."""
    rng = np.random.default_rng(7)
    K = 23
    t = rng.integers(-1, 2, (3, K)).astype(np.int8)
    want = []
    for row in t.tolist():
        digits = [v + 1 for v in row] + [1] * (-K % per)
        out = []
        for b in range(len(digits) // per):
            d = digits[b * per:(b + 1) * per]
            out.append(sum(u << (2 * i) for i, u in enumerate(d)) if fmt == "tq2" else sum(u * 3 ** i for i, u in enumerate(d)))
        want.append(out)
    assert orc.pack(t, fmt).tolist() == want


# ---- activation quantisation
def test_quant_act_int8_invariant_and_literals():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((5, 300)) * 3).astype(np.float32)
    q, s = orc.quant_act_int8(x)
    assert q.dtype == np.int8 and np.abs(q.astype(np.int32)).max() <= 127
    assert (np.abs(q.astype(np.float32) * s[:, None] - x) <= s[:, None] / 2 + 1e-6).all()
    # hand-computed: amax 254 -> s = 2; x / s = [127, -63.5, 0.5, 1.5, 2.5] -> half-to-even
    q, s = orc.quant_act_int8(np.array([[254.0, -127.0, 1.0, 3.0, 5.0]], np.float32))
    assert s.tolist() == [2.0] and q.tolist() == [[127, -64, 0, 2, 2]]
    q, s = orc.quant_act_int8(np.zeros((1, 4), np.float32))  # scale clamps at 1e-8
    assert s.tolist() == [np.float32(1e-8)] and not q.any()


# ---- GEMM reference
def _weights(E, N, K, group, fmt, seed=0):
    rng = np.random.default_rng(seed)
    trits = rng.integers(-1, 2, (E, N, K)).astype(np.int8)
    packed = np.stack([orc.pack(trits[e], fmt) for e in range(E)])
    scales = (rng.random((E, N, -(-K // group))).astype(np.float16).astype(np.float32) + np.float32(0.01))
    return trits, packed, scales


def _dense(x, xs, trits, scales, group):
    K = x.shape[1]
    w = trits.astype(np.float64) * np.repeat(scales.astype(np.float64), group, axis=1)[:, :K]
    return (x.astype(np.float64) * xs.astype(np.float64)[:, None]) @ w.T


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("K,group", [(256, 128), (300, 64), (130, 128)])
def test_reference_matches_dense(fmt, K, group):
    trits, packed, scales = _weights(1, 24, K, group, fmt)
    assert np.array_equal(orc.unpack(packed[0], fmt, K), trits[0])
    x, xs = orc.quant_act_int8(np.random.default_rng(1).standard_normal((5, K)).astype(np.float32))
    ref = orc.ternary_gemm_ref(x, xs, packed[0], scales[0], K, group, fmt)
    assert ref.dtype == np.float32
    np.testing.assert_allclose(ref, _dense(x, xs, trits[0], scales[0], group), rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_reference_integer_special_case(fmt):
    """scale = 1, one group, x_scale = 1: the contract reduces to an exact integer matmul."""
    rng = np.random.default_rng(3)
    K, N, M = 97, 11, 6
    t = rng.integers(-1, 2, (N, K)).astype(np.int8)
    x = rng.integers(-127, 128, (M, K)).astype(np.int8)
    out = orc.ternary_gemm_ref(x, np.ones(M, np.float32), orc.pack(t, fmt), np.ones((N, 1), np.float32), K, K, fmt)
    assert np.array_equal(out, (x.astype(np.int64) @ t.astype(np.int64).T).astype(np.float32))


def test_reference_group_order_and_rounding():
    """Two groups whose products do not commute in float32: pins 'multiply, add, in ascending g'."""
    K, group = 2, 1
    t = np.array([[1, 1]], np.int8)
    x = np.array([[127, -127]], np.int8)
    s = np.array([[np.float32(1.0000001), np.float32(1.0)]], np.float32)
    got = orc.ternary_gemm_ref(x, np.array([0.5], np.float32), orc.pack(t, "tq2"), s, K, group, "tq2")
    want = (np.float32(127) * s[0, 0] + np.float32(-127) * s[0, 1]) * np.float32(0.5)
    assert got[0, 0] == want and got[0, 0] != 0.0


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_float_contract_matches_dequantized(fmt):
    rng = np.random.default_rng(5)
    K, group, N = 200, 64, 37
    trits, packed, scales = _weights(1, N, K, group, fmt, seed=5)
    x = rng.standard_normal((4, K)).astype(np.float32)
    deq = orc.dequantize([(packed[0], scales[0])], K, group, fmt)
    np.testing.assert_allclose(orc.ternary_gemm_float_ref(x, packed[0], scales[0], K, group, fmt),
                               x.astype(np.float64) @ deq.astype(np.float64).T, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_grouped_matches_per_expert_and_routing_sort(fmt):
    E, N, K, group, T, k = 6, 16, 192, 64, 9, 2
    trits, packed, scales = _weights(E, N, K, group, fmt, seed=3)
    rng = np.random.default_rng(4)
    x, xs = orc.quant_act_int8(rng.standard_normal((T, K)).astype(np.float32))
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).reshape(-1)
    ids[ids == 5] = 4  # leave expert 5 empty
    order, offsets = orc.sort_by_expert(ids, E)
    assert offsets.tolist() == [0] + np.cumsum(np.bincount(ids, minlength=E)).tolist()
    assert sorted(order.tolist()) == list(range(T * k)) and (np.diff(ids[order]) >= 0).all()
    for e in range(E):  # stable: equal ids keep input order
        assert (np.diff(order[offsets[e]:offsets[e + 1]]) > 0).all()
    rows = order // k
    out = orc.grouped_ternary_gemm_ref(x[rows], xs[rows], offsets, packed, scales, K, group, fmt)
    for i, r in enumerate(rows.tolist()):
        e = int(ids[order[i]])
        want = orc.ternary_gemm_ref(x[r:r + 1], xs[r:r + 1], packed[e], scales[e], K, group, fmt)
        assert np.array_equal(out[i:i + 1], want)
    with pytest.raises(ValueError, match="offsets"):
        orc.grouped_ternary_gemm_ref(x, xs, [0, T], packed, scales, K, group, fmt)
    with pytest.raises(ValueError, match="unknown ternary packing"):
        orc.ternary_gemm_ref(x, xs, packed[0], scales[0], K, group, "tq3")


def test_bf16_rounding_helper():
    v = np.array([1.0, 1.00390625, 1.005859375, 1.01171875, -3.14159], np.float32)
    r = orc.bf16_round(v)
    # 1 + 2^-8 ties between 1.0 and 1 + 2^-7 -> even mantissa (1.0); 1 + 3*2^-9 rounds up to 1 + 2^-7;
    # 1 + 3*2^-8 ties between 1 + 2^-7 (odd) and 1 + 2^-6 (even) -> 1 + 2^-6
    assert r[:4].tolist() == [1.0, 1.0, 1.0078125, 1.015625]
    assert np.array_equal(orc.bf16_from_bits(orc.bf16_bits(v)), r)


def test_moe_layer_matches_per_token_dense():
    """moe_layer_ref against a per-token float64 evaluation of the same routed MLP."""
    rng = np.random.default_rng(11)
    H, I, E, k, T, group, fmt = 64, 32, 4, 2, 5, 32, "tq2"
    experts = []
    for e in range(E):
        mats = []
        for (n, kk) in ((I, H), (I, H), (H, I)):
            t = rng.integers(-1, 2, (n, kk)).astype(np.int8)
            s = (0.1 * np.abs(rng.standard_normal((n, kk // group)))).astype(np.float16)
            mats.append([(orc.pack(t, fmt), s)])
        experts.append(tuple(mats))
    x = orc.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    logits = rng.standard_normal((T, E)).astype(np.float32) * 1.5
    got = orc.moe_layer_ref(x, logits, experts, k, H, I, group, fmt, act="bf16")
    scores = orc.softmax_f32(logits)
    want = np.zeros((T, H))
    for t in range(T):
        top = np.argsort(-scores[t], kind="stable")[:k]
        for e in top:
            g, u, d = (orc.dequantize(m, kk, group, fmt).astype(np.float64) for m, kk in zip(experts[e], (H, H, I)))
            h = orc.silu(x[t] @ g.T) * (x[t] @ u.T)
            want[t] += (h @ d.T) * scores[t, e]
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 2e-2  # bf16 rounding at every stage


def test_absmean_ternary_known_answers():
    """The literal known-answer test of the reference (tests/test_qat.py:11-17: a short last group and an all-zero row),
    then cases that closed forms fix: small integers (every sum exact in any order), the clamp, ties to even."""
    w = np.array([[0.0, -2.0, 4.0, 3.0, -1.0], [0.0, 0.0, 0.0, 0.0, 0.0]], np.float32)
    trits, scale = orc.absmean_ternary(w, 3)
    assert np.array_equal(scale, np.array([[2.0, 2.0], [0.0, 0.0]], np.float32))
    assert np.array_equal(trits, np.array([[0, -1, 1, 1, 0], [0, 0, 0, 0, 0]], np.int8))
    # group mean 2: w / s = 0.5, 1.5, -0.5, -2.5 -> rint (ties to even) 0, 2, -0, -2 -> clamp 0, 1, 0, -1
    trits, scale = orc.absmean_ternary(np.array([[1.0, 3.0, -1.0, -5.0, 1.0, 1.0, 2.0, 2.0]], np.float32), 8)
    assert scale[0, 0] == 2.0 and np.array_equal(trits[0], [0, 1, 0, -1, 0, 0, 1, 1])
    # the scale is rounded to the stored format BEFORE the division: mean 1/3 -> fp16 0.33325195, bf16 0.333984375
    w = np.array([[1.0, 0.0, 0.0, 0.1666, 0.1667, 0.0]], np.float32)
    for dt, s in (("f16", np.float32(np.float16(1 / 3))), ("bf16", orc.bf16_round(np.array([1 / 3], np.float32))[0])):
        trits, scale = orc.absmean_ternary(w[:, :3], 3, dt)
        assert scale[0, 0] == s and np.array_equal(trits[0], [1, 0, 0])
    with pytest.raises(ValueError):
        orc.absmean_ternary(np.zeros((2, 0), np.float32), 3)
    with pytest.raises(ValueError):
        orc.absmean_ternary(np.zeros((2, 4), np.float32), 0)


# --------------------------------------------------------------------------- MoE oracles against torch CPU restatements
def _tiny_experts(rng, H, I, E, group, fmt, terms=1):
    experts = []
    for e in range(E):
        mats = []
        for (n, kk) in ((I, H), (I, H), (H, I)):
            ts = []
            for t in range(terms):
                tr = rng.integers(-1, 2, (n, kk)).astype(np.int8)
                sc = (0.1 * 0.25 ** t * np.abs(rng.standard_normal((n, kk // group)))).astype(np.float16)
                ts.append((orc.pack(tr, fmt), sc))
            mats.append(ts)
        experts.append(tuple(mats))
    return experts


def _torch_linear_bf16(x, terms, K, group, fmt):
    """A float-activation TernaryLinear on dequantized weights (boilerplate/ternary/ops.py:51-58, 81-86), the product in
    float64 so that its value is the exact one up to 2^-53, rounded to bf16 as ``out_dtype=x.dtype`` does."""
    import torch

    w = torch.from_numpy(orc.dequantize(terms, K, group, fmt).astype(np.float64))
    return (x.double() @ w.t()).float().to(torch.bfloat16)


def _bf16_ulps(a, b):
    """Distance in bf16 steps between two bf16-valued float32 arrays of one sign pattern (0 where equal)."""
    ia = (np.asarray(a, np.float32).view(np.uint32) >> 16).astype(np.int64)
    ib = (np.asarray(b, np.float32).view(np.uint32) >> 16).astype(np.int64)
    ia = np.where(ia & 0x8000, 0x8000 - ia, ia)
    ib = np.where(ib & 0x8000, 0x8000 - ib, ib)
    return np.abs(ia - ib)


@pytest.mark.parametrize("renorm", [False, True])
def test_moe_layer_ref_against_the_reference_lines_in_torch(renorm):
    """moe_layer_ref against boilerplate/engine/standard.py:151-176 restated line by line with torch CPU ops on bf16
    tensors (softmax, topk, F.silu, bf16 products, index_add_), the linears on dequantized weights. Every rounding
    point and the accumulation order are pinned: agreement within one bf16 step per element, nearly all equal."""
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(21)
    H, I, E, k, T, group, fmt = 64, 32, 6, 3, 40, 32, "tq1"
    experts = _tiny_experts(rng, H, I, E, group, fmt)
    x = orc.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    logits = (rng.standard_normal((T, E)) * 1.5).astype(np.float32)
    got = orc.moe_layer_ref(x, logits, experts, k, H, I, group, fmt, act="bf16", renorm=renorm)

    flat = torch.from_numpy(x).to(torch.bfloat16)
    scores = torch.softmax(torch.from_numpy(logits).float(), dim=-1)
    values, indices = torch.topk(scores, k, dim=-1)
    if renorm:
        values = values / values.sum(-1, keepdim=True)
    values = values.to(flat.dtype)
    output = torch.zeros_like(flat)
    for e in range(E):
        token, slot = torch.where(indices == e)
        if not token.numel():
            continue
        gate_t, up_t, down_t = experts[e]
        xe = flat[token]
        h = F.silu(_torch_linear_bf16(xe, gate_t, H, group, fmt)) * _torch_linear_bf16(xe, up_t, H, group, fmt)
        result = _torch_linear_bf16(h, down_t, I, group, fmt) * values[token, slot, None]
        output.index_add_(0, token, result.to(output.dtype))
    want = output.float().numpy()
    ulps = _bf16_ulps(got, want)
    assert ulps.max() <= 1, ulps.max()
    assert (ulps == 0).mean() >= 0.995, (ulps == 0).mean()


def test_topk_desc_matches_torch_topk():
    """The routing's top-k: values and indices equal torch.topk's on rows without ties (softmax scores of random logits), and
    on rows with ties the same VALUES; which of two equal scores torch.topk returns first is not specified by torch,
    the oracle takes the lower index (a stable sort)."""
    import torch

    rng = np.random.default_rng(5)
    scores = orc.softmax_f32((rng.standard_normal((200, 64)) * 1.5).astype(np.float32))
    assert all(np.unique(r).size == r.size for r in scores)
    v, i = orc.topk_desc(scores, 6)
    tv, ti = torch.topk(torch.from_numpy(scores), 6, dim=-1)
    assert np.array_equal(v, tv.numpy()) and np.array_equal(i, ti.numpy())
    tied = np.array([[0.25, 0.5, 0.25, 0.5, 0.125]], np.float32)
    v, i = orc.topk_desc(tied, 3)
    assert v.tolist() == [[0.5, 0.5, 0.25]] and i.tolist() == [[1, 3, 0]]
    assert torch.topk(torch.from_numpy(tied), 3).values.tolist() == v.tolist()


@pytest.mark.parametrize("limit", [0.0, 0.75])
def test_moe_layer_v4_ref_against_the_reference_lines_in_torch(limit):
    """moe_layer_v4_ref against boilerplate/engine/model.py:376-387 and :407-420 restated with torch CPU ops: bf16 linears
    widened to float32, the clamps, F.silu in float32, the routing weight before w2, one cast to bf16, float32 `y[idx] +=`.
    float32 silu differs from the oracle's correctly rounded one by an ulp now and then, which a bf16 rounding of the
    product rarely sees: within one bf16 step of w2's output scale, nearly all sums equal to the last float32 bit."""
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(22)
    H, I, E, k, T, group, fmt = 64, 32, 6, 3, 40, 32, "tq2"
    experts = _tiny_experts(rng, H, I, E, group, fmt, terms=2)
    x = orc.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    scores = orc.softmax_f32((rng.standard_normal((T, E)) * 1.5).astype(np.float32))
    _, indices = orc.topk_desc(scores, k)
    weights = (np.take_along_axis(scores, indices, -1) * np.float32(2.5)).astype(np.float32)  # (route_scale, model.py:404)
    got = orc.moe_layer_v4_ref(x, weights, indices, experts, H, I, group, fmt, act="bf16", swiglu_limit=limit)

    xt = torch.from_numpy(x).to(torch.bfloat16)
    wt, it = torch.from_numpy(weights), torch.from_numpy(indices)
    y = torch.zeros_like(xt, dtype=torch.float32)
    clamped = 0
    for e in range(E):
        idx, top = torch.where(it == e)
        if not idx.numel():
            continue
        w1, w3, w2 = experts[e]
        xe = xt[idx]
        gate, up = _torch_linear_bf16(xe, w1, H, group, fmt).float(), _torch_linear_bf16(xe, w3, H, group, fmt).float()
        if limit > 0:
            clamped += int((up.abs() > limit).sum() + (gate > limit).sum())
            up = torch.clamp(up, min=-limit, max=limit)
            gate = torch.clamp(gate, max=limit)
        h = F.silu(gate) * up
        h = wt[idx, top, None] * h
        y[idx] += _torch_linear_bf16(h.to(torch.bfloat16), w2, I, group, fmt)
    want = y.numpy()
    assert limit == 0 or clamped > 50  # the clamp is exercised
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= scale * 2.0 ** -7
    assert (got == want).mean() >= 0.98, (got == want).mean()
    # a dropped routing weight, a clamp on the wrong operand or bf16 accumulation would not pass:
    wrong = orc.moe_layer_v4_ref(x, np.ones_like(weights), indices, experts, H, I, group, fmt, swiglu_limit=limit)
    assert (wrong == want).mean() < 0.5


@pytest.mark.parametrize("sdt", ["f16", "bf16"])
def test_absmean_ternary_against_the_reference_formula_in_torch(sdt):
    """oracle.absmean_ternary against the literal formula of boilerplate/ternary/fit.py:84-95 evaluated with torch CPU ops
    (F.pad, abs().sum(-1) / counts, .to(scale_dtype), round, clamp) on Gaussian weights [256, 7168 + 40], group 128.
    `sum(-1)` leaves the order of the 128 float32 additions to the library (a vectorised cascade on the CPU, a tree on a
    GPU); the oracle and the HIP kernel add in ascending column order. The sums differ in their last float32 bit now and
    then, which moves a stored scale by one step of its format in about 2 in 10,000 groups (fp16; bf16: 1 in 10,000) and a
    trit next to a rounding boundary in fewer than 1 in a million. Measured here and bounded; everything else is equal."""
    import torch
    import torch.nn.functional as F

    g = torch.Generator().manual_seed(0)
    W = torch.randn(256, 7168 + 40, generator=g) * 0.02
    group, dt = 128, {"f16": torch.float16, "bf16": torch.bfloat16}[sdt]
    rows, columns = W.shape
    groups = -(-columns // group)
    data = F.pad(W.float(), (0, groups * group - columns)).view(rows, groups, group)
    counts = torch.full((groups,), group, dtype=torch.float32)
    counts[-1] = columns - (groups - 1) * group
    scale = (data.abs().sum(-1) / counts).to(dt)
    sf = scale.float().unsqueeze(-1)
    trits = torch.where(sf > 0, torch.round(data / sf.clamp_min(1e-30)).clamp(-1, 1), 0).to(torch.int8).view(rows, -1)[:, :columns]
    to, so = orc.absmean_ternary(W.numpy(), group, sdt)
    want_s = scale.float().numpy()
    step = np.abs(want_s) * (2.0 ** -10 if sdt == "f16" else 2.0 ** -7)
    assert (np.abs(so - want_s) <= step).all()          # never more than one step of the stored format
    assert (so != want_s).mean() <= 1e-3, (so != want_s).mean()
    assert (to != trits.numpy()).mean() <= 1e-5, (to != trits.numpy()).mean()
    # the short last group divides by its own count (40), not by 128
    assert np.allclose(so[:, -1], np.abs(W.numpy()[:, -40:]).sum(1) / 40, rtol=2e-2)

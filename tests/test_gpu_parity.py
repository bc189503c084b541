"""Parity of the HIP path (through the C ABI, via the Python mirror) against the CPU oracle.

Bars: decoded trits, packed bytes, scales, int8 activations and routing indices bit-exact; GEMM
outputs within rel-L2 <= 1e-3 (and max-abs <= 2e-2 on bf16 outputs) of the CPU oracle, plus the
reference's own backend tolerances (rtol 1e-4 / atol 1e-3, reference tests/test_ternary_cuda.py:80,87)
on its test shapes; the reference-order kernel bit-exact on the int8 path.
"""

import itertools

import numpy as np
import pytest
import torch

from _util import c_gemm, golden, orc, rel_l2, synth_trits, synth_weights

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3  # north-star tolerance vs the CPU ternary kernel
MAX_ABS_BF16 = 2e-2


@pytest.fixture(scope="module")
def bp():
    import deepseekternarized_amd as m

    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    assert m.ext() is not None, "the HIP extension must load on a GPU box (no fallback)"
    return m


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def bf16_dev(a):
    return dev(np.asarray(a, np.float32)).to(torch.bfloat16)


# --------------------------------------------------------------------------- formats: bit-exact
@pytest.mark.parametrize("fmt", ["tq2", "tq1"])
@pytest.mark.parametrize("K", [1, 4, 5, 7, 128, 131, 640, 4099])
def test_pack_unpack_bit_exact(bp, fmt, K):
    rng = np.random.default_rng(K)
    t = rng.integers(-1, 2, (9, K)).astype(np.int8)
    p = bp.pack(dev(t), fmt)
    assert p.dtype == torch.uint8 and tuple(p.shape) == (9, bp.packed_cols(fmt, K))
    assert np.array_equal(p.cpu().numpy(), orc.pack(t, fmt))
    assert np.array_equal(bp.unpack(p, fmt, K).cpu().numpy(), t)


@pytest.mark.parametrize("fmt", ["tq2", "tq1"])
@pytest.mark.parametrize("K", [16, 5120, 5136, 7168, 20496])
def test_pack_unpack_in_16_byte_pieces_bit_exact(bp, fmt, K):
    """K a multiple of 16: the kernels that move the trit side in 16-byte pieces through LDS, a workgroup per 1024 packed
    bytes of a row - one segment, a segment that ends inside a TQ1 byte's five trits, several segments per row."""
    rng = np.random.default_rng(K)
    t = rng.integers(-1, 2, (37, K)).astype(np.int8)
    p = bp.pack(dev(t), fmt)
    assert np.array_equal(p.cpu().numpy(), orc.pack(t, fmt))
    assert np.array_equal(bp.unpack(p, fmt, K).cpu().numpy(), t)
    if K == 16:  # more rows than one grid dimension's second extent holds
        tall = rng.integers(-1, 2, (70001, K)).astype(np.int8)
        pt = bp.pack(dev(tall), fmt)
        assert np.array_equal(pt.cpu().numpy(), orc.pack(tall, fmt))
        assert np.array_equal(bp.unpack(pt, fmt, K).cpu().numpy(), tall)
    # every byte value on the unpack side (TQ2 code 3 -> +2, TQ1 bytes >= 243 -> 0), rows of other lengths around it
    raw = rng.integers(0, 256, (5, bp.packed_cols(fmt, K))).astype(np.uint8)
    assert np.array_equal(bp.unpack(dev(raw), fmt, K).cpu().numpy(), orc.unpack(raw, fmt, K))


@pytest.mark.parametrize("fmt", ["tq2", "tq1"])
def test_unpack_every_byte_value_bit_exact(bp, fmt):
    """All 256 byte values, incl. TQ2 code 3 (-> +2) and TQ1 bytes >= 243 (-> 0)."""
    per = 4 if fmt == "tq2" else 5
    p = np.arange(256, dtype=np.uint8).reshape(1, 256)
    for K in (256 * per, 256 * per - 2):
        got = bp.unpack(dev(p), fmt, K).cpu().numpy()
        assert np.array_equal(got, orc.unpack(p, fmt, K))


def test_tq1_every_pattern_and_lut(bp):
    pats = np.array(list(itertools.product([-1, 0, 1], repeat=5)), dtype=np.int8)
    p = bp.pack(dev(pats), "tq1").cpu().numpy()
    assert np.unique(p).size == 243 and int(p.max()) < 243
    assert np.array_equal(bp.tq1_lut("cuda").cpu().numpy(), orc.tq1_lut())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_scale_expansion_bit_exact(bp, dtype):
    from deepseekternarized_amd.ternary.pack import expand_scales

    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)  # every 16-bit pattern
    got = expand_scales(bits.cuda()).cpu()
    want = bits.float()
    assert torch.equal(got.view(torch.int32)[~want.isnan()], want.view(torch.int32)[~want.isnan()])
    assert bool(got[want.isnan()].isnan().all())


@pytest.mark.parametrize("K", [300, 64, 2048, 8192, 8200])  # rows of whole 16-byte pieces up to 8192 take the one-read kernel (16-bit inputs)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_quant_act_int8_bit_exact(bp, dtype, K):
    rng = np.random.default_rng(K)
    x = torch.from_numpy((rng.standard_normal((37, K)) * 3).astype(np.float32)).to(dtype)
    x[3] = 0  # scale clamps at 1e-8
    x[4, :5] = torch.tensor([254.0, -127.0, 1.0, 3.0, 5.0]).to(dtype)
    q, s = bp.quant_act_int8(x.cuda())
    wq, ws = orc.quant_act_int8(x.float().numpy())
    assert q.dtype == torch.int8 and s.dtype == torch.float32 and tuple(s.shape) == (37,)
    assert np.array_equal(s.cpu().numpy(), ws) and np.array_equal(q.cpu().numpy(), wq)
    assert ((q.float() * s[:, None] - x.cuda().float()).abs() <= s[:, None] / 2 + 1e-6).all()
    # A NaN makes its row's scale NaN, an infinity makes it infinite (the int8 values of such a row are a cast of NaN in
    # the reference, boilerplate/ternary/ops.py:22: unspecified); the other rows are not touched by it.
    y = x.clone()
    y[1, K // 2] = float("nan")
    y[2, K - 1] = float("inf")
    q2, s2 = bp.quant_act_int8(y.cuda())
    keep = np.array([r not in (1, 2) for r in range(37)])
    assert np.array_equal(q2.cpu().numpy()[keep], wq[keep]) and np.array_equal(s2.cpu().numpy()[keep], ws[keep])
    assert np.isnan(s2[1].item()) and np.isinf(s2[2].item())


def test_quant_act_int8_keeps_leading_shape(bp):
    x = torch.randn(3, 5, 64, generator=torch.Generator().manual_seed(0))
    q, s = bp.quant_act_int8(x.cuda())
    assert tuple(q.shape) == (3, 5, 64) and tuple(s.shape) == (3, 5)


# --------------------------------------------------------------------------- routing: bit-exact
@pytest.mark.parametrize("n,E", [(0, 4), (1, 1), (18, 6), (6, 64), (100, 384), (128, 3), (129, 7), (64, 5000), (512, 384), (4096, 64), (12288, 384),
                                  (70000, 8), (3000, 5000), (2048, 1), (2048, 4096), (2049, 64), (1500, 4097),
                                  (777, 2500)])  # up to 128 ids: the one-pass kernel
def test_sort_by_expert_bit_exact(bp, n, E):
    rng = np.random.default_rng(n + E)
    ids = rng.integers(0, E, n).astype(np.int64)
    if n > 10:
        ids[ids == E - 1] = 0  # leave the last expert empty
    order, offsets = bp.sort_by_expert(dev(ids), E)
    worder, woffsets = orc.sort_by_expert(ids, E)
    assert np.array_equal(offsets.cpu().numpy(), woffsets)
    assert np.array_equal(order.cpu().numpy(), worder)  # stable: identical to argsort(kind="stable")


def test_gather_rows_bit_exact(bp):
    from deepseekternarized_amd.kernels.ternary_hip import gather_rows

    rng = np.random.default_rng(1)
    for cols, dtype in ((4096, torch.bfloat16), (36, torch.int8), (130, torch.float32)):
        src = torch.from_numpy(rng.integers(-100, 100, (17, cols)).astype(np.float32)).to(dtype)
        order = torch.from_numpy(rng.permutation(17 * 6).astype(np.int64))
        got = gather_rows(src.cuda(), order.cuda(), 6).cpu()
        assert torch.equal(got, src[order // 6])


@pytest.mark.parametrize("rows,inter", [(37, 2048), (5, 1028), (3, 1030), (70000, 8)])
def test_swiglu_bit_exact(bp, rows, inter):
    """h = bf16(bf16(silu(bf16 gate)) * bf16 up), the expert MLP's elementwise stage (boilerplate/engine/standard.py:151-154),
    against torch on bf16 tensors: four columns per thread where the row length allows it, one otherwise (1030), more
    rows than a grid's y extent."""
    from deepseekternarized_amd.moe import swiglu_bf16

    g = torch.Generator(device="cuda").manual_seed(rows + inter)
    gu = torch.randn(rows, 2 * inter, device="cuda", generator=g) * 3.0
    got = swiglu_bf16(gu, inter)
    gate, up = gu[:, :inter].to(torch.bfloat16), gu[:, inter:].to(torch.bfloat16)
    want = torch.nn.functional.silu(gate) * up
    assert got.dtype == torch.bfloat16 and torch.equal(got, want)


# --------------------------------------------------------------------------- GEMM vs golden fixtures
def _lin_terms(c):
    return [dev(c[f"packed{t}"]) for t in range(c["terms"])], [dev(c[f"scale{t}"]) for t in range(c["terms"])]


@pytest.mark.parametrize("backend", ["auto", "torch"])
@pytest.mark.parametrize("name", sorted(golden()))
def test_gemm_matches_reference_cpu_kernel_fixture(bp, name, backend):
    """Outputs of the reference's compiled CPU kernel (tests/golden/ref_cpu_kernel.npz) on its own test shapes."""
    c = golden()[name]
    pk, sc = _lin_terms(c)
    if c["int8"]:
        got = bp.ternary_gemm(dev(c["x"]), dev(c["x_scale"]), pk, sc, c["K"], c["group"], c["fmt"], backend=backend)
    else:
        got = bp.ternary_gemm_float(dev(c["x"]), pk, sc, c["K"], c["group"], c["fmt"], backend=backend)
    got = got.cpu().numpy()
    np.testing.assert_allclose(got, c["out"], rtol=1e-4, atol=1e-3)
    assert rel_l2(got, c["out"]) <= REL_L2


@pytest.mark.parametrize("name", [n for n in sorted(golden()) if golden()[n]["int8"]])
def test_reference_order_kernel_is_bit_exact(bp, name):
    """backend="torch" follows kernels/ternary_cuda.py:52-64 operation for operation."""
    c = golden()[name]
    pk, sc = _lin_terms(c)
    got = bp.ternary_gemm_ref(dev(c["x"]), dev(c["x_scale"]), pk[0], sc[0], c["K"], c["group"], c["fmt"]).cpu().numpy()
    want = orc.ternary_gemm_ref(c["x"], c["x_scale"], c["packed0"], c["scale0"].astype(np.float32), c["K"], c["group"], c["fmt"])
    assert np.array_equal(got, want)


# --------------------------------------------------------------------------- GEMM vs oracle, seeded
def _check(got, want, bf16_out=False):
    got = np.asarray(got, np.float64)
    assert np.isfinite(got).all()
    assert rel_l2(got, want) <= REL_L2, rel_l2(got, want)
    if bf16_out:
        assert np.abs(got - want).max() <= MAX_ABS_BF16


@pytest.mark.parametrize("fmt", ["tq2", "tq1"])
@pytest.mark.parametrize("M", [1, 8])
def test_config0_single_linear_fp32_activations(bp, fmt, M):
    """K=4096, N=2048, fp32 activations, M in {1, 8} against the CPU kernel port."""
    N, K, group = 2048, 4096, 128
    packed, scales = synth_weights(0, 1, N, K, group, fmt)
    x = np.random.default_rng(100 + M).standard_normal((M, K)).astype(np.float32)
    want = c_gemm(x, None, packed[0][0], scales[0][0].astype(np.float32), K, group, fmt)
    got = bp.ternary_gemm_float(dev(x), dev(packed[0][0]), dev(scales[0][0]), K, group, fmt).cpu().numpy()
    _check(got, want)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("N,K", [(2048, 7168), (7168, 2048)])
@pytest.mark.parametrize("M", [1, 4, 16, 32])
def test_config1_decode_gemv_bf16(bp, fmt, N, K, M):
    group = 128
    packed, scales = synth_weights(1, 1, N, K, group, fmt)
    x = orc.bf16_round(np.random.default_rng(M).standard_normal((M, K)).astype(np.float32))
    want = c_gemm(x, None, packed[0][0], scales[0][0].astype(np.float32), K, group, fmt)
    lin = bp.TernaryLinear([bp.PackedTerm(dev(packed[0][0]), dev(scales[0][0]))], K, fmt, group, act="bf16")
    y32 = lin(bf16_dev(x), out_dtype=torch.float32).cpu().numpy()
    _check(y32, want)
    ybf = lin(bf16_dev(x)).float().cpu().numpy()  # default out_dtype bf16
    assert np.abs(ybf - want).max() <= MAX_ABS_BF16


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("M", [1, 16, 32])
def test_config1_decode_gemv_int8(bp, fmt, M):
    """Mode D activations (per-row int8) at config-1 size. K = 7168 is not a multiple of the K chunk the
    kernels stage for 16 token rows, so the last chunk is a short one."""
    N, K, group = 2048, 7168, 128
    packed, scales = synth_weights(2, 1, N, K, group, fmt)
    x = np.random.default_rng(40 + M).standard_normal((M, K)).astype(np.float32)
    q, qs = orc.quant_act_int8(x)
    want = c_gemm(q, qs, packed[0][0], scales[0][0].astype(np.float32), K, group, fmt)
    got = bp.ternary_gemm(dev(q), dev(qs), dev(packed[0][0]), dev(scales[0][0]), K, group, fmt).cpu().numpy()
    _check(got, want)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("act", ["int8", "bf16"])
@pytest.mark.parametrize("K,group", [(256, 128), (640, 128), (200, 64), (1024, 256)])
def test_ternary_linear_stacked_terms(bp, fmt, act, K, group):
    """Reference tests/test_ternary.py:85-98: N=37, x [3, 5, K] bf16, k=2 terms."""
    N = 37
    packed, scales = synth_weights(K, 1, N, K, group, fmt, terms=2)
    terms = [bp.PackedTerm(dev(p[0]), dev(s[0])) for p, s in zip(packed, scales)]
    x = orc.bf16_round(np.random.default_rng(K).standard_normal((3, 5, K)).astype(np.float32))
    got = bp.TernaryLinear(terms, K, fmt, group, act=act)(bf16_dev(x), out_dtype=torch.float32)
    assert tuple(got.shape) == (3, 5, N)
    want = orc.ternary_linear_ref(x, [(p[0], s[0]) for p, s in zip(packed, scales)], K, group, fmt, act).reshape(3, 5, N)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("T", [1, 3, 37])
def test_grouped_reference_cuda_acceptance_shapes(bp, fmt, T):
    """Reference tests/test_ternary_cuda.py:69-87: E=5, N=70, K=4160, counts [T, 0, 2T, 1, T]."""
    E, N, K, group = 5, 70, 4160, 128
    packed, scales = synth_weights(7, E, N, K, group, fmt)
    counts = np.array([T, 0, 2 * T, 1, T])
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    x, xs = orc.quant_act_int8(np.random.default_rng(9).standard_normal((int(offsets[-1]), K)).astype(np.float32))
    want = orc.grouped_ternary_gemm_ref(x, xs, offsets, packed[0], scales[0].astype(np.float32), K, group, fmt)
    got = bp.grouped_ternary_gemm(dev(x), dev(xs), offsets.tolist(), dev(packed[0]), dev(scales[0]), K, group, fmt)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=1e-3)
    got_dev = bp.grouped_ternary_gemm(dev(x), dev(xs), dev(offsets), dev(packed[0]), dev(scales[0]).float(), K, group, fmt)
    assert torch.equal(got, got_dev)  # device offsets (no host copy) and f32 scales give the same result


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_grouped_with_routing_sort_and_bad_offsets(bp, fmt):
    """Reference tests/test_ternary_cuda.py:41-57: E=6, N=16, K=192, g=64, T=9, top-2, one empty expert."""
    E, N, K, group, T, k = 6, 16, 192, 64, 9, 2
    packed, scales = synth_weights(3, E, N, K, group, fmt)
    rng = np.random.default_rng(4)
    x, xs = orc.quant_act_int8(rng.standard_normal((T, K)).astype(np.float32))
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).reshape(-1)
    ids[ids == 5] = 4
    order, offsets = bp.sort_by_expert(dev(ids), E)
    rows = order // k
    out = bp.grouped_ternary_gemm(dev(x)[rows], dev(xs)[rows], offsets, dev(packed[0]), dev(scales[0]), K, group, fmt)
    worder, woffsets = orc.sort_by_expert(ids, E)
    want = orc.grouped_ternary_gemm_ref(x[worder // k], xs[worder // k], woffsets, packed[0], scales[0].astype(np.float32), K, group, fmt)
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-4)
    with pytest.raises(ValueError, match="offsets"):
        bp.grouped_ternary_gemm(dev(x), dev(xs), [0, T], dev(packed[0]), dev(scales[0]), K, group, fmt)


def test_native_boundary_rejects_malformed_tensors(bp):
    """Reference tests/test_kernel_security.py:19-38 restated for the device module: every malformed
    tensor raises RuntimeError before any kernel runs."""
    e = bp.ext()

    def args():
        return dict(out=torch.zeros(1, 2, device="cuda"), x=torch.ones(1, 5, dtype=torch.int8, device="cuda"),
                    x_scale=torch.ones(1, device="cuda"), offsets=torch.tensor([0, 1], device="cuda"),
                    packed=torch.ones(1, 2, 2, dtype=torch.uint8, device="cuda"), w_scale=torch.ones(1, 2, 2, device="cuda"),
                    K=5, group=3, fmt=2, lut1=None, max_rows=1)

    e.ternary_grouped_gemm(*args().values())  # the well-formed call passes
    bad = [("K", 0), ("K", 2 ** 62), ("group", 0), ("fmt", 0),
           ("x", torch.ones(1, 4, dtype=torch.int8, device="cuda")), ("x", torch.ones(1, 5, dtype=torch.float64, device="cuda")),
           ("out", torch.zeros(1, 1, device="cuda")), ("out", torch.zeros(1, 2, dtype=torch.float64, device="cuda")),
           ("packed", torch.ones(1, 2, 1, dtype=torch.uint8, device="cuda")), ("packed", torch.ones(1, 2, 2, device="cuda")),
           ("w_scale", torch.ones(1, 2, 1, device="cuda")), ("w_scale", torch.ones(1, 1, 2, device="cuda")),
           ("x_scale", torch.ones(0, device="cuda")), ("lut1", torch.ones(1, dtype=torch.int8, device="cuda")),
           ("packed", torch.ones(1, 2, 4, dtype=torch.uint8, device="cuda")[:, :, ::2]),
           ("offsets", torch.tensor([0, 1, 1], device="cuda")), ("out", torch.zeros(1, 2)), ("max_rows", -1)]
    for key, value in bad:
        a = args()
        a[key] = value
        with pytest.raises(RuntimeError):
            e.ternary_grouped_gemm(*a.values())


def test_accumulates_into_out(bp):
    """The native entry adds into `out` (ternary_cuda_kernel.cu:96), so stacked terms can share one buffer."""
    e = bp.ext()
    N, K, group = 32, 256, 128
    packed, scales = synth_weights(5, 1, N, K, group, "tq2")
    x, xs = orc.quant_act_int8(np.random.default_rng(5).standard_normal((3, K)).astype(np.float32))
    out = torch.full((3, N), 2.5, device="cuda")
    e.ternary_grouped_gemm(out, dev(x), dev(xs), torch.tensor([0, 3], device="cuda"), dev(packed[0]), dev(scales[0]), K, group, 2)
    want = 2.5 + orc.ternary_gemm_ref(x, xs, packed[0][0], scales[0][0].astype(np.float32), K, group, "tq2")
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_empty_and_ragged_inputs(bp, fmt):
    K, group, N = 131, 64, 5
    packed, scales = synth_weights(2, 3, N, K, group, fmt)
    x0 = torch.zeros(0, K, dtype=torch.int8, device="cuda")
    out = bp.grouped_ternary_gemm(x0, torch.zeros(0, device="cuda"), [0, 0, 0, 0], dev(packed[0]), dev(scales[0]), K, group, fmt)
    assert tuple(out.shape) == (0, N)
    x, xs = orc.quant_act_int8(np.random.default_rng(3).standard_normal((4, K)).astype(np.float32))
    offsets = [0, 0, 4, 4]  # only the middle expert has rows
    got = bp.grouped_ternary_gemm(dev(x), dev(xs), offsets, dev(packed[0]), dev(scales[0]), K, group, fmt)
    want = orc.grouped_ternary_gemm_ref(x, xs, offsets, packed[0], scales[0].astype(np.float32), K, group, fmt)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-4)


# --------------------------------------------------------------------------- configs 2 and 3 (full shapes)
def _route(rng, T, E, k):
    logits = (rng.standard_normal((T, E)) * 1.5).astype(np.float32)
    scores = orc.softmax_f32(logits)
    _, idx = orc.topk_desc(scores, k)
    return logits, idx.astype(np.int64)


@pytest.fixture(scope="module")
def cfg2_weights(bp):
    E, N, K, group, fmt = 64, 2048, 4096, 128, "tq1"
    rng = np.random.default_rng(2)
    trits = synth_trits(rng, (E, N, K))
    scale = (0.02 * np.abs(rng.standard_normal((E, N, K // group)))).astype(np.float16)
    packed = bp.pack(dev(trits.reshape(E * N, K)), fmt).view(E, N, -1)
    return trits, scale, packed


@pytest.mark.parametrize("T,bound", [(1, None), (32, None), (32, 32), (40, 40), (256, None)])
def test_config2_grouped_tq1_full_shape_sampled(bp, cfg2_weights, T, bound):
    """64 experts, gate projection 2048 x 4096 TQ1, top-6 skewed routing; every routed row checked on a
    sample of output columns against the float64 oracle (the full oracle product would take minutes).
    `bound`: max_rows as the MoE layer passes it for a few tokens (the token count, an upper bound on the widest
    expert's rows, so that nothing is read back): the call then runs as launches of 8 rows per expert."""
    from deepseekternarized_amd.kernels.ternary_hip import gather_rows

    E, N, K, group, k, fmt = 64, 2048, 4096, 128, 6, "tq1"
    trits, scale, packed = cfg2_weights
    rng = np.random.default_rng(T)
    x = orc.bf16_round(rng.standard_normal((T, K)).astype(np.float32))
    _, idx = _route(rng, T, E, k)
    order, offsets = bp.sort_by_expert(dev(idx.reshape(-1)), E)
    xg = gather_rows(bf16_dev(x), order, k)
    got = bp.grouped_ternary_gemm(xg, None, offsets, packed, dev(scale), K, group, fmt, max_rows=bound).cpu().numpy()
    if bound is not None:
        assert bp.ext().last_kernel().startswith("fp4_tq1_m"), bp.ext().last_kernel()
    worder, woffsets = orc.sort_by_expert(idx.reshape(-1), E)
    assert np.array_equal(order.cpu().numpy(), worder)
    cols = rng.choice(N, 48, replace=False)
    want = np.zeros((T * k, cols.size))
    for e in range(E):
        a, b = int(woffsets[e]), int(woffsets[e + 1])
        if a < b:
            w = trits[e][cols].astype(np.float64) * np.repeat(scale[e][cols].astype(np.float64), group, axis=1)
            want[a:b] = x[worder[a:b] // k].astype(np.float64) @ w.T
    _check(got[:, cols], want)


def test_config3_grouped_tq2_two_terms_sampled(bp):
    """Stacked residual k=2 (second-term scales 0.25x), TQ2, top-6 of 384 experts (E reduced to 48 and
    T to 256 so the weights fit a test; per-expert row counts keep the same ~32-row skewed profile)."""
    E, N, K, group, k, fmt, T = 48, 2048, 4096, 128, 6, "tq2", 256
    rng = np.random.default_rng(33)
    trits = [synth_trits(rng, (E, N, K)) for _ in range(2)]
    s0 = (0.02 * np.abs(rng.standard_normal((E, N, K // group)))).astype(np.float16)
    scales = [s0, (s0.astype(np.float32) * 0.25).astype(np.float16)]
    packed = [bp.pack(dev(t.reshape(E * N, K)), fmt).view(E, N, -1) for t in trits]
    x = orc.bf16_round(rng.standard_normal((T, K)).astype(np.float32))
    _, idx = _route(rng, T, E, k)
    order, offsets = bp.sort_by_expert(dev(idx.reshape(-1)), E)
    from deepseekternarized_amd.kernels.ternary_hip import gather_rows

    xg = gather_rows(bf16_dev(x), order, k)
    got = bp.grouped_ternary_gemm(xg, None, offsets, packed, [dev(s) for s in scales], K, group, fmt).cpu().numpy()
    worder, woffsets = orc.sort_by_expert(idx.reshape(-1), E)
    cols = rng.choice(N, 32, replace=False)
    want = np.zeros((T * k, cols.size))
    for e in range(E):
        a, b = int(woffsets[e]), int(woffsets[e + 1])
        if a < b:
            w = sum(t[e][cols].astype(np.float64) * np.repeat(s[e][cols].astype(np.float64), group, axis=1)
                    for t, s in zip(trits, scales))
            want[a:b] = x[worder[a:b] // k].astype(np.float64) @ w.T
    _check(got[:, cols], want)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_linearity_at_full_size(bp, fmt):
    """Size-independent property at config-1 size: f(a x1 + b x2) = a f(x1) + b f(x2) for exactly
    representable combinations, and f(e_k) reads out column k of the dequantized weight."""
    N, K, group = 2048, 7168, 128
    rng = np.random.default_rng(8)
    trits = synth_trits(rng, (N, K))
    scale = (0.02 * np.abs(rng.standard_normal((N, K // group)))).astype(np.float16)
    packed = bp.pack(dev(trits), fmt)
    x1 = orc.bf16_round(rng.integers(-8, 9, (2, K)).astype(np.float32))
    x2 = orc.bf16_round(rng.integers(-8, 9, (2, K)).astype(np.float32))
    f = lambda x: bp.ternary_gemm_float(bf16_dev(x), packed, dev(scale), K, group, fmt).cpu().numpy().astype(np.float64)
    np.testing.assert_allclose(f(2 * x1 - x2), 2 * f(x1) - f(x2), rtol=1e-4, atol=1e-4)
    ks = [0, 1, 127, 128, 129, 639, 640, 641, K - 1]
    eye = np.zeros((len(ks), K), np.float32)
    eye[np.arange(len(ks)), ks] = 1.0
    want = (trits[:, ks].astype(np.float32) * scale[:, [k // group for k in ks]].astype(np.float32)).T
    assert np.array_equal(f(eye).astype(np.float32), want)  # one nonzero product per output: exact


# --------------------------------------------------------------------------- MoE layer (engine call pattern)
@pytest.mark.parametrize("fmt,act", [("tq1", "bf16"), ("tq2", "bf16"), ("tq2", "int8")])
def test_moe_layer_matches_reference_call_pattern(bp, fmt, act):
    """route -> per-expert SwiGLU -> weighted combine with the rounding points of
    boilerplate/engine/standard.py:151-176, against oracle.moe_layer_ref (top-2 of 8 experts, one empty)."""
    from deepseekternarized_amd.moe import TernaryMoE

    H, I, E, k, T, group = 1024, 1024, 8, 2, 12, 128
    rng = np.random.default_rng(21)
    mats = {}
    for name, (n, kk) in (("gate", (I, H)), ("up", (I, H)), ("down", (H, I))):
        tr = synth_trits(rng, (E, n, kk))
        sc = (0.05 * np.abs(rng.standard_normal((E, n, kk // group)))).astype(np.float16)
        mats[name] = (np.stack([orc.pack(tr[e], fmt) for e in range(E)]), sc)
    x = orc.bf16_round(rng.standard_normal((T, H)).astype(np.float32))
    logits = (rng.standard_normal((T, E)) * 1.5).astype(np.float32)
    logits[:, 5] = -30.0  # expert 5 is never routed to
    experts = [tuple([(mats[n][0][e], mats[n][1][e])] for n in ("gate", "up", "down")) for e in range(E)]
    want = orc.moe_layer_ref(x, logits, experts, k, H, I, group, fmt, act=act)
    moe = TernaryMoE(*[[(dev(mats[n][0]), dev(mats[n][1]))] for n in ("gate", "up", "down")], H, I, k, fmt, group, act=act)
    got = moe(bf16_dev(x), dev(logits)).float().cpu().numpy()
    assert got.shape == (T, H) and np.isfinite(got).all()
    # both sides round to bf16 at the same points; float32 summation order may flip a few roundings
    assert rel_l2(got, want) <= 5e-3, rel_l2(got, want)
    assert np.abs(got - want).max() <= MAX_ABS_BF16 * max(1.0, np.abs(want).max())


# --------------------------------------------------------------------------- producer: absmean quantizer + packer
def test_absmean_known_answer_of_the_reference(bp):
    """reference tests/test_qat.py:11-17, literally: a short last group and an all-zero row."""
    weight = torch.tensor([[0.0, -2.0, 4.0, 3.0, -1.0], [0.0, 0.0, 0.0, 0.0, 0.0]], device="cuda")
    result = bp.absmean_ternary(weight, group=3)
    assert torch.equal(result.scale.cpu(), torch.tensor([[2.0, 2.0], [0.0, 0.0]], dtype=torch.float16))
    assert torch.equal(result.trits.cpu(), torch.tensor([[0, -1, 1, 1, 0], [0, 0, 0, 0, 0]], dtype=torch.int8))
    with pytest.raises(ValueError):
        bp.absmean_ternary(weight, group=0)
    with pytest.raises(ValueError):
        bp.absmean_ternary(weight, group=3, scale_dtype=torch.float32)
    with pytest.raises(ValueError):
        bp.packed_term(weight, 3, "tq3")


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sdtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("K,group", [(131, 64), (640, 128), (4099, 256), (7, 3)])
def test_absmean_and_packed_term_bit_exact(bp, wdtype, sdtype, K, group):
    """Trits, scales and packed bytes bit-identical to the oracle (same float32 summation order), and
    packed_term == pack(absmean trits) for both formats (boilerplate/qat/bitlinear.py:75-80)."""
    rng = np.random.default_rng(K + group)
    w = rng.standard_normal((37, K)).astype(np.float32) * np.exp(rng.uniform(-3, 3, (37, 1))).astype(np.float32)
    w[5] = 0.0
    w[6, : K // 2] = 0.0
    wt = dev(w).to(wdtype)
    w_seen = wt.float().cpu().numpy()
    want_trits, want_scale = orc.absmean_ternary(w_seen, group, "f16" if sdtype == torch.float16 else "bf16")
    term = bp.absmean_ternary(wt, group, sdtype)
    assert term.scale.dtype == sdtype and term.trits.dtype == torch.int8
    assert np.array_equal(term.scale.float().cpu().numpy(), want_scale)
    assert np.array_equal(term.trits.cpu().numpy(), want_trits)
    for fmt in ("tq1", "tq2"):
        pt = bp.packed_term(wt, group, fmt, sdtype)
        assert np.array_equal(pt.packed.cpu().numpy(), orc.pack(want_trits, fmt))
        assert torch.equal(pt.scale, term.scale)


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K,group", [(7168, 128), (7168, 256), (2048, 96), (1000, 100), (256, 1000), (4096, 4096)])
def test_absmean_with_the_row_staged_in_lds_bit_exact(bp, wdtype, K, group):
    """Rows of whole 16-byte pieces: the producer reads its row once into LDS. Groups that end inside a 16-byte piece, a
    last group shorter than the others, one group longer than the row: scales, trits and packed bytes bit-identical to
    the oracle (group sums in ascending k)."""
    rng = np.random.default_rng(K + group)
    w = rng.standard_normal((21, K)).astype(np.float32) * np.exp(rng.uniform(-3, 3, (21, 1))).astype(np.float32)
    w[3] = 0.0
    w[4, K // 3:] = 0.0
    wt = dev(w).to(wdtype)
    w_seen = wt.float().cpu().numpy()
    want_trits, want_scale = orc.absmean_ternary(w_seen, group, "f16")
    term = bp.absmean_ternary(wt, group, torch.float16)
    assert np.array_equal(term.scale.float().cpu().numpy(), want_scale)
    assert np.array_equal(term.trits.cpu().numpy(), want_trits)
    for fmt in ("tq1", "tq2"):
        pt = bp.packed_term(wt, group, fmt, torch.float16)
        assert np.array_equal(pt.packed.cpu().numpy(), orc.pack(want_trits, fmt))
        assert torch.equal(pt.scale, term.scale)


@pytest.mark.parametrize("sdtype", [torch.float16, torch.bfloat16])
def test_absmean_weights_at_the_rounding_boundary(bp, sdtype):
    """Weights within a few units in the last place of half their group's scale, where rint(w / s) changes between 0 and
    +-1 (a quotient of exactly 1/2 rounds to even, 0): the producer decides without dividing, the oracle divides. Groups
    of 128 whose mean is a power of two (so that the stored scale is the mean exactly), at magnitudes from 2^-20 to 2^10,
    and a group of NaN / infinite weights."""
    rng = np.random.default_rng(99)
    N, K, group = 64, 1024, 128
    w = np.zeros((N, K), np.float32)
    for n in range(N):
        for g in range(K // group):
            s = np.float32(2.0) ** int(rng.integers(-20, 11))
            half = np.float32(0.5) * s
            near = (np.full(64, half, np.float32).view(np.int32) + rng.integers(-3, 4, 64).astype(np.int32)).view(np.float32)
            near *= rng.choice(np.array([-1, 1], np.float32), 64)
            # the other 64 weights make the group's mean |w| exactly s: each pair (near, 2 s - |near|) sums to 2 s
            rest = (2 * s - np.abs(near)).astype(np.float32) * rng.choice(np.array([-1, 1], np.float32), 64)
            w[n, g * group:(g + 1) * group] = rng.permutation(np.concatenate([near, rest]))
    w[3, :group] = np.nan
    w[4, 5] = np.inf
    w[5, :group] = 0.0
    wt = dev(w)
    with np.errstate(invalid="ignore"):  # (the NaN and infinite weights of rows 3 and 4)
        want_trits, want_scale = orc.absmean_ternary(w, group, "f16" if sdtype == torch.float16 else "bf16")
    term = bp.absmean_ternary(wt, group, sdtype)
    assert np.array_equal(term.scale.float().cpu().numpy(), want_scale, equal_nan=True)
    assert np.array_equal(term.trits.cpu().numpy(), want_trits)
    assert (np.abs(want_trits[8:]) == 0).mean() > 0.1 and (np.abs(want_trits[8:]) == 1).mean() > 0.5  # (both sides of the boundary occur)


def test_packed_term_feeds_the_linear_like_the_training_graph(bp):
    """reference tests/test_qat.py:52-59 (BitLinear training graph == packed engine), K=131, group 64: the packed term
    made on the device, run through TernaryLinear, equals the dequantized product."""
    rng = np.random.default_rng(52)
    K, N, group = 131, 24, 64
    w = dev(rng.standard_normal((N, K)).astype(np.float32))
    x = bf16_dev(rng.standard_normal((5, K)).astype(np.float32))
    for fmt in ("tq1", "tq2"):
        lin = bp.TernaryLinear([bp.packed_term(w, group, fmt)], K, fmt, group, act="int8")
        q, s = bp.quant_act_int8(x)
        want = (q.float() * s[:, None]) @ lin.dequantized().t()
        got = lin(x, out_dtype=torch.float32)
        torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-3)


# --------------------------------------------------------------------------- operator-layer pieces of the reference interface
@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_dequantized_matches_the_reference_formula(bp, fmt):
    """boilerplate/ternary/ops.py:51-58: sum over terms of unpack(packed).float() * scale.float().repeat_interleave(group)[:, :K]."""
    N, K, group = 37, 200, 64
    packed, scales = synth_weights(9, 1, N, K, group, fmt, terms=2)
    lin = bp.TernaryLinear([bp.PackedTerm(dev(p[0]), dev(s[0])) for p, s in zip(packed, scales)], K, fmt, group)
    want = None
    for p, s in zip(packed, scales):
        d = orc.unpack(p[0], fmt, K).astype(np.float32) * np.repeat(s[0].astype(np.float32), group, axis=1)[:, :K]
        want = d if want is None else want + d
    got = lin.dequantized()
    assert got.dtype == torch.float32 and got.is_cuda and np.array_equal(got.cpu().numpy(), want)
    assert lin.dequantized() is got  # kept


def test_module_level_tq1_table(bp):
    from deepseekternarized_amd.ternary.pack import _TQ1_LUT

    t = _TQ1_LUT.to("cuda")
    assert t.dtype == torch.int8 and tuple(t.shape) == (256, 5) and np.array_equal(t.cpu().numpy(), orc.tq1_lut())
    assert _TQ1_LUT.to("cuda") is t


def test_sort_by_expert_ids_out_of_range(bp):
    """Ids outside [0, E): left out of the count by default (documented divergence: the reference's bincount raises for
    negative ids); `validate=True` raises."""
    ids = torch.tensor([3, 0, 7, -1, 2, 8, 0], device="cuda")
    order, offsets = bp.sort_by_expert(ids, 8)
    assert offsets.cpu().tolist() == [0, 2, 2, 3, 4, 4, 4, 4, 5]
    assert order.cpu().tolist()[:5] == [1, 6, 4, 0, 2]
    with pytest.raises(ValueError):
        bp.sort_by_expert(ids, 8, validate=True)
    order, offsets = bp.sort_by_expert(ids.clamp(0, 7), 8, validate=True)
    assert offsets.cpu().tolist()[-1] == 7 and sorted(order.cpu().tolist()) == list(range(7))


def test_max_rows_bound_too_small_is_reported_on_request(bp):
    """Device offsets with a caller's bound: rows beyond it are left out without an error (documented); `validate=True`
    raises the reference's message (ternary_cuda_kernel.cu:130-139 checks a host copy on every call)."""
    E, N, K, group = 3, 16, 256, 128
    packed, scales = synth_weights(5, E, N, K, group, "tq2")
    rng = np.random.default_rng(6)
    x, xs = orc.quant_act_int8(rng.standard_normal((9, K)).astype(np.float32))
    offsets = torch.tensor([0, 5, 5, 9], device="cuda")
    full = bp.grouped_ternary_gemm(dev(x), dev(xs), offsets, dev(packed[0]), dev(scales[0]), K, group, "tq2", max_rows=5, validate=True)
    with pytest.raises(RuntimeError, match="max_rows is smaller"):
        bp.grouped_ternary_gemm(dev(x), dev(xs), offsets, dev(packed[0]), dev(scales[0]), K, group, "tq2", max_rows=4, validate=True)
    part = bp.grouped_ternary_gemm(dev(x), dev(xs), offsets, dev(packed[0]), dev(scales[0]), K, group, "tq2", max_rows=4)
    assert torch.equal(part[:4], full[:4]) and torch.equal(part[5:9], full[5:9]) and not part[4].any()  # expert 0's fifth row is left at zero

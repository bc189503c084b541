"""Seeded random grouped calls against the CPU oracle: formats, activation and scale dtypes, 1 - 4 stacked terms, scale
groups of 128 / 256, host or device offsets with tight or loose row bounds, heavy-tailed activations, and operand
tensors that start at other addresses than an allocation's (activations and scales moved by whole 16-byte pieces, TQ1
packed bytes by any number of bytes). Which kernel a case runs on is the dispatcher's choice; the draw covers every
tuned kernel family and the general one (the test asserts that it did)."""

import numpy as np
import pytest
import torch

from _util import c_gemm, orc, rel_l2, synth_weights

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _shifted(t, elems):
    """A copy of t that starts `elems` elements into a 64-byte aligned allocation, with other values around it."""
    buf = torch.full((t.numel() + 64,), 3, dtype=t.dtype, device="cuda")
    base = ((64 - buf.data_ptr() % 64) % 64) // t.element_size() + elems
    buf[base:base + t.numel()] = t.reshape(-1)
    return buf[base:base + t.numel()].view(t.shape)


def _case(bp, seed):
    rng = np.random.default_rng(seed)
    fmt = str(rng.choice(["tq1", "tq2"]))
    group = int(rng.choice([128, 128, 256]))
    K = int(rng.choice([1024, 1280, 1536, 2048, 2304, 2560, 3072, 4096, 5120, 5376, 7168, 8192]))
    N = int(rng.choice([16, 48, 64, 144, 512, 1040, 2048, 2064]))
    E = int(rng.choice([1, 2, 3, 5]))
    hi = int(rng.choice([1, 2, 8, 20, 40, 70]))
    counts = [int(rng.integers(0, hi + 1)) for _ in range(E)]
    if sum(counts) == 0:
        counts[-1] = 1
    act = str(rng.choice(["bf16", "int8", "f16", "f32"], p=[0.4, 0.4, 0.1, 0.1]))
    terms = int(rng.choice([1, 2, 3, 4]))
    sdt = str(rng.choice(["f16", "bf16", "f32"], p=[0.6, 0.25, 0.15]))
    packed, scales = synth_weights(seed, E, N, K, group, fmt, terms=terms)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    T = int(offsets[-1])
    x = rng.standard_normal((T, K)).astype(np.float32)
    if rng.random() < 0.3:
        x *= np.exp(rng.standard_normal((T, K)) * 2).astype(np.float32)
    xs = None
    if act == "int8":
        x, xs = orc.quant_act_int8(x)
        xd, xsd = dev(x), dev(xs)
    elif act == "bf16":
        x = orc.bf16_round(x)
        xd, xsd = dev(x).to(torch.bfloat16), None
    elif act == "f16":
        x = x.astype(np.float16).astype(np.float32)
        xd, xsd = dev(x).half(), None
    else:
        xd, xsd = dev(x), None
    if sdt == "f16":
        sc, sref = [dev(s) for s in scales], [s.astype(np.float32) for s in scales]
    elif sdt == "f32":
        sc, sref = [dev(s.astype(np.float32)) for s in scales], [s.astype(np.float32) for s in scales]
    else:
        sc = [dev(s.astype(np.float32)).to(torch.bfloat16) for s in scales]
        sref = [t.float().cpu().numpy() for t in sc]
    pk = [dev(p) for p in packed]
    if rng.random() < 0.3:
        xd = _shifted(xd, 16 * int(rng.integers(1, 4)))
    if rng.random() < 0.3:
        e_ = int(rng.choice([2, 4, 8, 16]))
        sc = [_shifted(s, e_) for s in sc]
    if rng.random() < 0.3:
        e_ = 16 if fmt == "tq2" else int(rng.integers(1, 17))
        pk = [_shifted(p, e_) for p in pk]
    want = np.zeros((T, N), np.float32)
    for e in range(E):
        a, b = int(offsets[e]), int(offsets[e + 1])
        for p, s in zip(packed, sref):
            if b > a:
                c_gemm(x[a:b], None if xs is None else xs[a:b], p[e], s[e], K, group, fmt, out=want[a:b])
    if rng.random() < 0.5:
        got = bp.grouped_ternary_gemm(xd, xsd, offsets.tolist(), pk, sc, K, group, fmt)
    else:
        bound = int(max(counts)) if rng.random() < 0.5 else T
        got = bp.grouped_ternary_gemm(xd, xsd, torch.from_numpy(offsets).cuda(), pk, sc, K, group, fmt, max_rows=bound)
    return got.cpu().numpy(), want, bp.ext().last_kernel()


def test_seeded_random_grouped_calls():
    import deepseekternarized_amd as bp

    families = set()
    for seed in range(7000, 7100):
        got, want, kernel = _case(bp, seed)
        assert np.isfinite(got).all(), (seed, kernel)
        assert rel_l2(got, want) <= 1e-3, (seed, kernel, rel_l2(got, want))
        families.add(kernel.split("_")[0] + "_" + kernel.split("_")[1])
    assert {"general_float", "general_i8", "fp4_tq1", "gemm_tq1", "gemm_tq1f", "gemm_tq2", "mfma_tq1", "mfma_tq2"} <= families, families

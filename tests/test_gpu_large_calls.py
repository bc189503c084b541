"""Large calls: the tuned kernels chosen for launches that fill the device (16-wave variants, the K-split and streaming
decode GEMVs, tile kernels) against the library's general kernel, which keeps the reference's operation order
(boilerplate/kernels/ternary_cuda.py:52-64) and is itself checked against the CPU kernel in test_gpu_parity.py. The CPU
kernel would take minutes on these sizes; the weights are drawn and packed on the device."""
import pytest
import torch

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3  # per output row, float32 sums against float32 sums


@pytest.fixture(scope="module")
def bp():
    import deepseekternarized_amd as bp_

    if bp_.ext() is None:
        pytest.fail("HIP extension missing on a GPU box")
    return bp_


@pytest.mark.parametrize("fmt", ["tq2", "tq1"])
@pytest.mark.parametrize("E,N,K", [(64, 2048, 7168), (48, 1536, 4096), (32, 7168, 2048)])
@pytest.mark.parametrize("group,scale_dtype,terms,acts", [(128, torch.float16, 1, ("bf16", "int8")),
                                                          (256, torch.float32, 2, ("bf16", "int8", "f16", "f32")),
                                                          (128, torch.bfloat16, 2, ("bf16", "f32"))])
def test_tuned_kernels_of_large_calls_agree_with_the_general_kernel(bp, fmt, E, N, K, group, scale_dtype, terms, acts):
    g = torch.Generator(device="cuda").manual_seed(E + N)
    packed = torch.empty(E, N, bp.packed_cols(fmt, K), dtype=torch.uint8, device="cuda")
    for e in range(E):
        packed[e] = bp.pack(torch.randint(-1, 2, (N, K), device="cuda", generator=g).to(torch.int8), fmt)
    scale = (0.02 * torch.randn(E, N, K // group, device="cuda", generator=g).abs()).half().to(scale_dtype)
    packed, scale = [packed] * terms, [scale * 0.5 ** t for t in range(terms)]  # (the terms share their trits: what is checked is the sum)
    seen = set()
    for act in acts:
        for rows, ragged in [(1, False), (2, False), (3, False), (4, False), (5, False), (6, False), (7, False), (8, False),
                             (9, False), (11, False), (14, False), (16, True), (17, True), (33, True)]:
            counts = [rows] * E
            if rows > 1:  # (every third expert a row short; ragged: the first expert takes those rows and is the widest)
                for e in range(1, E, 3):
                    counts[e] -= 1
                    counts[0] += 1 if ragged else 0
            offsets = [0]
            for c in counts:
                offsets.append(offsets[-1] + c)
            T = offsets[-1]
            if act != "int8":
                x, xs = torch.randn(T, K, device="cuda", generator=g).to({"bf16": torch.bfloat16, "f16": torch.float16, "f32": torch.float32}[act]), None
            else:
                x = torch.randint(-127, 128, (T, K), device="cuda", generator=g).to(torch.int8)
                xs = torch.rand(T, device="cuda", generator=g) * 0.01 + 0.001
            got = bp.grouped_ternary_gemm(x, xs, offsets, packed, scale, K, group, fmt)
            kern = bp.ext().last_kernel()
            ref = bp.grouped_ternary_gemm(x, xs, offsets, packed, scale, K, group, fmt, backend="torch")
            assert bp.ext().last_kernel() != kern, kern
            assert torch.isfinite(got).all(), (act, rows, kern)
            err = ((got.double() - ref.double()).norm(dim=1) / ref.double().norm(dim=1).clamp_min(1e-30)).max().item()
            assert err <= REL_L2, (act, rows, kern, err)
            seen.add(kern)
    assert len(seen) >= 4, seen  # (decode GEMV, small-batch and tile kernels all took part)

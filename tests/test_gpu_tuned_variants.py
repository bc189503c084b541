"""Every code path of the tuned kernels (bp_mfma_tq2.hip, bp_tq2_gemv_fp4.hip, bp_gemm_tq2.hip, bp_mfma_tq1.hip, bp_gemm_tq1.hip, bp_tq1_gemv.hip, bp_tq1_gemv_fp4.hip) against the CPU oracle.

The shapes are chosen by what they select inside the launchers, not by size: odd / even packed row
lengths (row starts at every byte alignment), K that fits one activation / table tile or needs several,
scales through the LDS tile or - misaligned, or too many groups - from global memory, one or two stacked
terms, every activation dtype, empty experts, N not a multiple of the rows of a workgroup.
"""

import numpy as np
import pytest
import torch

from _util import c_gemm, orc, rel_l2, synth_weights

pytestmark = pytest.mark.gpu

REL_L2 = 1e-3
GROUP = 128


@pytest.fixture(scope="module")
def bp():
    import deepseekternarized_amd as m

    assert torch.cuda.is_available() and m.ext() is not None
    return m


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _activations(rng, T, K, act):
    x = rng.standard_normal((T, K)).astype(np.float32)
    if act == "int8":
        q, s = orc.quant_act_int8(x)
        return q, s, dev(q), dev(s)
    if act == "bf16":
        x = orc.bf16_round(x)
        return x, None, dev(x).to(torch.bfloat16), None
    if act == "f16":
        x = x.astype(np.float16).astype(np.float32)
        return x, None, dev(x).half(), None
    return x, None, dev(x), None


def _run(bp, fmt, E, N, K, counts, act, terms=1, seed=0, misalign_scales=False, scale_dtype=np.float16, group=GROUP, max_rows=None):
    """Grouped call with `counts[e]` rows per expert; returns (got, want, kernel name). `max_rows`: offsets on the
    device and that upper bound, as a caller that does not read the counts back passes them."""
    rng = np.random.default_rng(seed)
    packed, scales = synth_weights(seed, E, N, K, group, fmt, terms=terms)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    T = int(offsets[-1])
    x, xs, xd, xsd = _activations(rng, T, K, act)
    want = np.zeros((T, N), np.float32)
    for e in range(E):
        a, b = int(offsets[e]), int(offsets[e + 1])
        for p, s in zip(packed, scales):
            if b > a:
                c_gemm(x[a:b], None if xs is None else xs[a:b], p[e], s[e].astype(np.float32), K, group, fmt, out=want[a:b])
    pk = [dev(p) for p in packed]
    if scale_dtype is np.float16:
        sc = [dev(s) for s in scales]
    elif scale_dtype == "f32":  # the stored fp16 values widened, as the reference's wrappers pass them
        sc = [dev(s.astype(np.float32)) for s in scales]
    else:
        sc = [dev(s.astype(np.float32)).to(torch.bfloat16) for s in scales]
        # the oracle must see the rounded scales
        want[:] = 0
        for e in range(E):
            a, b = int(offsets[e]), int(offsets[e + 1])
            for p, s in zip(packed, sc):
                if b > a:
                    c_gemm(x[a:b], None if xs is None else xs[a:b], p[e], s[e].float().cpu().numpy(), K, group, fmt, out=want[a:b])
    if misalign_scales:  # a view whose data pointer is 4- but not 16-byte aligned
        moved = []
        for s in sc:
            flat = torch.empty(s.numel() + 2, dtype=s.dtype, device="cuda")
            flat[2:].copy_(s.reshape(-1))
            moved.append(flat[2:].view(s.shape))
            assert moved[-1].data_ptr() % 16 == 4
        sc = moved
    if max_rows is None:
        got = bp.grouped_ternary_gemm(xd, xsd, offsets.tolist(), pk, sc, K, group, fmt)  # host offsets: max_rows = widest expert
    else:
        got = bp.grouped_ternary_gemm(xd, xsd, torch.from_numpy(offsets).cuda(), pk, sc, K, group, fmt, max_rows=max_rows)
    return got.cpu().numpy(), want, bp.ext().last_kernel()


def _check(got, want):
    assert np.isfinite(got).all()
    assert rel_l2(got, want) <= REL_L2, rel_l2(got, want)


# --------------------------------------------------------------------------- TQ1 decode GEMV
# Three kernels: fp8 x fp4 matrix instructions with every wave walking along its own rows (16-bit and int8 activations,
# tables that fit in LDS), the same instructions with the rows streamed through LDS tile by tile and a chunk of the
# token's operand per wave (large calls; BP_TUNE_TQ1=chunk selects it wherever it can run, =rows never), and the table
# lookup of partial sums (everything else; BP_TUNE_TQ1=lut selects it for every call; the `tune` fixture makes the
# library read the switch again).
@pytest.fixture(params=["fp4", "chunk", "lut"])
def gemv_kernel(request, tune):
    tune("BP_TUNE_TQ1", {"fp4": "rows", "chunk": "chunk", "lut": "lut"}[request.param])
    return "lut_tq1" if request.param == "lut" else "fp4_tq1"


@pytest.mark.parametrize("K", [1024, 1280, 2048, 4352, 7168])  # Kp = 205 (odd: rows at every byte alignment), 256, 410, 871, 1434
@pytest.mark.parametrize("act", ["bf16", "int8"])
def test_tq1_gemv_row_alignments_and_tiles(bp, K, act, gemv_kernel):
    got, want, kern = _run(bp, "tq1", 3, 48, K, [1, 0, 1], act, seed=K)
    assert kern.startswith(gemv_kernel), kern
    _check(got, want)


@pytest.mark.parametrize("act,prefix", [("f16", "fp4_tq1"), ("f32", "lut_tq1")])
def test_tq1_gemv_other_activation_dtypes(bp, act, prefix, gemv_kernel):
    got, want, kern = _run(bp, "tq1", 2, 32, 2048, [1, 1], act, seed=3)
    assert kern.startswith(prefix if gemv_kernel == "fp4_tq1" else "lut_tq1"), kern
    _check(got, want)


def test_tq1_gemv_many_rows_two_terms_bf16_scales(bp, gemv_kernel):
    """N spans several workgroups and is not a multiple of their rows; two stacked terms; bf16 scales."""
    got, want, kern = _run(bp, "tq1", 2, 2048 + 48, 2304, [1, 1], "bf16", terms=2, seed=5, scale_dtype=np.float32)
    assert kern.startswith(gemv_kernel), kern
    _check(got, want)


@pytest.mark.parametrize("act", ["bf16", "int8", "f16"])
@pytest.mark.parametrize("K,N,counts,terms,scale_dtype,group,misalign", [
    (1024, 48, [1, 0, 1], 1, np.float16, 128, False),    # 2 chunks: six of the eight waves have none
    (5376, 2048, [1], 2, "bf16", 128, False),            # 9 chunks: 2, 2, 2, 2, 1, 0, 0, 0 per wave; two terms = two rounds of the sum through LDS
    (7168, 2048, [0, 1], 2, np.float16, 256, False),     # 12 chunks, one scale per 256
    (2304, 528, [1, 1, 1], 1, np.float16, 128, True),    # scales from global memory (misaligned rows of scales); N not a multiple of 128
    (4608, 4096, [1], 1, "f32", 128, False),             # float32 scales: not this variant
])
def test_tq1_single_token_call_with_few_row_tiles_splits_the_chunks_over_the_waves(bp, act, K, N, counts, terms, scale_dtype, group, misalign):
    """One token and no more row tiles than CUs (a dense linear of a decode step): a row tile per workgroup, its chunks
    split over the 8 waves, partial sums added in wave order (kernel name fp4_tq1_t1_ks)."""
    got, want, kern = _run(bp, "tq1", len(counts), N, K, counts, act, terms=terms, seed=K + N, scale_dtype=scale_dtype, group=group,
                           misalign_scales=misalign)
    if scale_dtype != "f32":
        assert kern == "fp4_tq1_t1_ks", kern
    else:
        assert kern.startswith("fp4_tq1_t1_w"), kern
    _check(got, want)
    if act != "f16":  # the same call twice gives the same bits (fixed order of the waves' sums)
        again, _, _ = _run(bp, "tq1", len(counts), N, K, counts, act, terms=terms, seed=K + N, scale_dtype=scale_dtype, group=group,
                           misalign_scales=misalign)
        assert np.array_equal(got, again)


@pytest.mark.parametrize("K,counts,act,N", [(1024, [1, 0, 1], "bf16", 48),      # Kp = 205: rows at every byte alignment; 2 chunks, 5 groups of waves
                                           (1280, [1, 1], "int8", 2048 + 16),   # Kp = 256; N not a multiple of a workgroup's tiles
                                           (4352, [0, 1, 1], "f16", 80),        # 7 chunks: one group, 9 loaders
                                           (7168, [1, 1, 1], "bf16", 2048),     # 12 chunks, 4 loaders: the decode shape
                                           (7680, [1, 1], "int8", 96)])         # 12 chunks of rows of 1536 bytes: 7 wave loads per loader
def test_tq1_gemv_chunk_per_wave(bp, tune, K, counts, act, N):
    """The kernel that streams the rows through LDS tile by tile: every split of the 16 waves into groups, multipliers
    and loaders; odd and even row lengths; empty experts; the token's tile aliasing the tile buffers."""
    tune("BP_TUNE_TQ1", "chunk")
    got, want, kern = _run(bp, "tq1", len(counts), N, K, counts, act, seed=K + 1)
    assert kern == "fp4_tq1_t1_cw", kern
    _check(got, want)


def test_tq1_gemv_chunk_per_wave_terms_scales_groups(bp, tune):
    """Two stacked terms with bf16 scales (the second term adds to the first one's output), scale groups of 256, float32
    scales (what the reference's wrappers pass: boilerplate/kernels/ternary_cuda.py:95-97), and the calls it leaves to
    the other kernels: 15 chunks or more."""
    tune("BP_TUNE_TQ1", "chunk")
    got, want, kern = _run(bp, "tq1", 2, 2048 + 48, 2304, [1, 1], "bf16", terms=2, seed=5, scale_dtype=np.float32)
    assert kern == "fp4_tq1_t1_cw", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 3, 272, 2560, [1, 1, 1], "bf16", terms=2, seed=9, group=256)
    assert kern == "fp4_tq1_t1_cw", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 2, 64, 2048, [1, 1], "bf16", seed=10, scale_dtype="f32")
    assert kern == "fp4_tq1_t1_cw", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 3, 2048 + 16, 7168, [1, 0, 1], "int8", terms=2, seed=11, scale_dtype="f32")  # four wave loads of scales per tile
    assert kern == "fp4_tq1_t1_cw", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 2, 272, 4608, [2, 1], "bf16", seed=14, scale_dtype="f32", group=256)  # a pair of rows
    assert kern == "fp4_tq1_m2_cw", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 1, 272, 10240, [1], "bf16", seed=12)  # 16 chunks: no wave left for the loads
    assert kern.startswith("fp4_tq1_t1_w"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 2, 96, 9472, [1, 1], "int8", seed=13)  # 15 chunks: one loader, three wave loads of scales
    assert kern.startswith("fp4_tq1_t1_w"), kern
    _check(got, want)


@pytest.mark.parametrize("K,counts,act", [(1024, [2, 0, 1], "bf16"), (7168, [2, 2, 1], "int8"), (2304, [1, 2], "bf16"), (4352, [2, 2], "int8")])
def test_tq1_gemv_chunk_per_wave_token_pairs(bp, tune, K, counts, act):
    """The same kernel with a pair of token rows per expert (two fp8 pieces per activation, one matrix instruction for both
    tokens): experts with two rows, one row and none; two stacked terms; N not a multiple of a workgroup's tiles."""
    tune("BP_TUNE_TQ1", "chunk")
    got, want, kern = _run(bp, "tq1", len(counts), 2048 + 48, K, counts, act, terms=2, seed=K + 2)
    assert kern == "fp4_tq1_m2_cw", kern
    _check(got, want)


@pytest.mark.parametrize("K,counts,act", [(1024, [4, 0, 3], "bf16"), (7168, [4, 3, 1], "int8"), (2304, [3, 4], "bf16"), (4352, [4, 4], "int8"),
                                          (7168, [4, 4, 4], "bf16")])
def test_tq1_gemv_chunk_per_wave_four_rows(bp, tune, K, counts, act):
    """The same kernel with up to four token rows per expert: a matrix instruction per 16-byte piece of a row (80
    consecutive digits, at most two scale groups), operand rows = 2 group slots x 4 tokens x 2 pieces, four accumulator
    tiles per chunk; experts with four, three, one and no rows; two stacked terms; N not a multiple of a workgroup's tiles."""
    tune("BP_TUNE_TQ1", "chunk")
    got, want, kern = _run(bp, "tq1", len(counts), 2048 + 48, K, counts, act, terms=2, seed=K + 4)
    assert kern == "fp4_tq1_m4_cw", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", len(counts), 272, K, counts, act, seed=K + 5, scale_dtype=np.float16, group=256 if K % 512 == 0 and K >= 2048 else 128)
    assert kern == "fp4_tq1_m4_cw", kern
    _check(got, want)


def test_tq1_gemv_chunk_per_wave_pair_after_launches_of_eight(bp, tune):
    """Up to 10 rows per expert where most experts have few: a launch of 8 rows, then the rows 8 and 9 as a pair."""
    tune("BP_TUNE_TQ1", "chunk")
    got, want, kern = _run(bp, "tq1", 8, 272, 2048, [10, 1, 0, 2, 1, 0, 9, 1], "bf16", seed=17)
    assert kern == "fp4_tq1_m2_cw", kern
    _check(got, want)


def test_tq1_gemv_chunk_per_wave_random_shapes(bp, tune):
    """30 seeded random calls with one or two rows per expert (experts, rows, K, activation type, terms, scale type and
    group size drawn at random, some experts empty): whatever kernel takes them, the oracle decides; most land on the
    kernel under test."""
    tune("BP_TUNE_TQ1", "chunk")
    rng = np.random.default_rng(123)
    on_it = 0
    for it in range(30):
        E, N, K = int(rng.integers(1, 7)), 16 * int(rng.integers(1, 40)), 256 * int(rng.integers(1, 31))
        M, act, terms = int(rng.integers(1, 3)), ["bf16", "int8"][int(rng.integers(0, 2))], int(rng.integers(1, 3))
        group = 128 if K % 512 or rng.integers(0, 2) else 256
        counts = [int(rng.integers(0, M + 1)) for _ in range(E)]
        counts[-1] = M
        got, want, kern = _run(bp, "tq1", E, N, K, counts, act, terms=terms, seed=1000 + it, group=group,
                               scale_dtype=[np.float16, np.float32][int(rng.integers(0, 2))])
        on_it += kern.endswith("_cw")
        assert np.isfinite(got).all() and rel_l2(got, want) <= REL_L2, (it, E, N, K, counts, act, terms, group, kern, rel_l2(got, want))
    assert on_it >= 20, on_it


def test_tq1_fp4_small_batches_many_rows_bf16_scales(bp):
    """The small-batch variants over several workgroups and row blocks (N not a multiple of their rows), bf16 scales,
    int8 activations with their per-row scales."""
    for counts, act, want_kernel in [([2, 1], "bf16", "fp4_tq1_m2"), ([3, 4], "int8", "fp4_tq1_m4"), ([8, 5], "bf16", "fp4_tq1_m8")]:
        got, want, kern = _run(bp, "tq1", 2, 2048 + 48, 2304, counts, act, terms=2, seed=6, scale_dtype=np.float32)
        assert kern.startswith(want_kernel), kern
        _check(got, want)


def test_tq1_gemv_scales_from_global_memory(bp, tune):
    """Table kernel: scale pointers that are not 16-byte aligned, and K with more groups than the LDS tile takes."""
    tune("BP_TUNE_TQ1", "lut")
    got, want, kern = _run(bp, "tq1", 2, 32, 2048, [1, 1], "bf16", seed=6, misalign_scales=True)
    assert kern.startswith("lut_tq1") and kern.endswith("_gs"), kern
    _check(got, want)
    tune("BP_TUNE_TQ1", None)
    got, want, kern = _run(bp, "tq1", 2, 32, 2048, [1, 1], "bf16", seed=6, misalign_scales=True)
    assert kern.startswith("fp4_tq1"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 1, 272, 40960, [1], "bf16", seed=7)  # 64 chunks: the operand tile does not fit in LDS
    assert kern.startswith("lut_tq1"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 1, 272, 16384, [1], "bf16", seed=8)  # 26 chunks: one workgroup of 16 waves per CU
    assert kern == "fp4_tq1_t1_w16", kern
    _check(got, want)


@pytest.mark.parametrize("act", ["bf16", "f16"])
def test_tq1_gemv_fp8_pieces_keep_small_activations(bp, act):
    """The fp8 x fp4 kernel splits an activation into three E4M3 pieces under a per-group power-of-two prescale;
    what it drops is below 2^-20 of the largest magnitude of the 128-wide group. Activations spread over 5 decades,
    with outliers 1000 x the typical value, must still come out far inside the tolerance of the other paths."""
    rng = np.random.default_rng(11)
    E, N, K = 2, 64, 4352
    packed, scales = synth_weights(11, E, N, K, GROUP, "tq1")
    x = rng.standard_normal((E, K)).astype(np.float32) * np.exp(rng.uniform(-6, 6, (E, K))).astype(np.float32)
    x[:, ::97] *= 1000.0
    x = orc.bf16_round(x) if act == "bf16" else np.clip(x, -6e4, 6e4).astype(np.float16).astype(np.float32)
    want = np.zeros((E, N), np.float32)
    for e in range(E):
        c_gemm(x[e:e + 1], None, packed[0][e], scales[0][e].astype(np.float32), K, GROUP, "tq1", out=want[e:e + 1])
    xd = dev(x).to(torch.bfloat16) if act == "bf16" else dev(x).half()
    got = bp.grouped_ternary_gemm(xd, None, [0, 1, 2], [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq1").cpu().numpy()
    assert bp.ext().last_kernel().startswith("fp4_tq1")
    assert rel_l2(got, want) <= 1e-4, rel_l2(got, want)  # (measured 4e-5; the other paths are held to 1e-3)
    z = np.zeros_like(x)  # all-zero activations: the prescale has nothing to go by
    got = bp.grouped_ternary_gemm(dev(z).to(torch.bfloat16), None, [0, 1, 2], [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq1")
    assert torch.equal(got, torch.zeros_like(got))


# --------------------------------------------------------------------------- TQ1 grouped GEMM (token tiles of 32) and the 16-token MFMA kernel
@pytest.fixture(params=["gemm", "mfma"])
def tq1_rows_kernel(request, tune):
    """More than 8 rows per expert: the fp8 x fp4 grouped GEMM; BP_TUNE_TQ1=mfma keeps the older 16-token kernel covered."""
    tune("BP_TUNE_TQ1", "mfma" if request.param == "mfma" else None)
    return request.param + "_tq1"


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K", [1024, 2048, 7168])
@pytest.mark.parametrize("counts", [[2, 0, 5], [16, 3, 1], [20, 1, 37]])
def test_tq1_mfma_tiles(bp, K, counts, act, tq1_rows_kernel):
    got, want, kern = _run(bp, "tq1", 3, 80, K, counts, act, terms=2, seed=K + sum(counts))
    # (up to 8 rows per expert go to the small-batch fp8 x fp4 kernel)
    assert kern.startswith(tq1_rows_kernel if max(counts) > 6 or tq1_rows_kernel == "mfma_tq1" else "fp4_tq1_m6"), kern
    _check(got, want)


@pytest.fixture(params=["staged", "inline"])
def tq1_gemm_kernel(request, tune):
    """More than 8 rows per expert, bf16 activations: the grouped GEMM over activations converted into a workspace, one
    matrix instruction per scale group (kernel name gemm_tq1f_bf16; the default with a workspace, which the mirrored call
    brings), and the kernel that converts them itself (gemm_tq1_bf16; BP_TUNE_TQ2G=bf16 or no workspace). int8 activations
    run gemm_tq1_i8 either way."""
    tune("BP_TUNE_TQ2G", "fp4" if request.param == "staged" else "bf16")
    return "gemm_tq1f_bf16" if request.param == "staged" else "gemm_tq1_bf16"


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize(
    "E,N,K,counts,terms",
    [
        (3, 80, 1280, [33, 0, 64], 1),          # Kp = 256: every row dword-aligned; exactly two chunks; full 32-token tiles and a 1-token one
        (5, 528, 2048, [20, 1, 37, 9, 32], 2),   # two row blocks, the second with 16 of its 512 rows; Kp = 410: rows at two byte alignments
        (11, 48, 4096, [17] * 11, 1),            # more experts than XCDs and not a multiple of 8; 7 chunks, the last one with 2 groups (its second window is skipped)
        (2, 1040, 7168, [48, 31], 1),            # config-1 K: 12 chunks, the last one with a single group; three row blocks
        (3, 64, 1024, [9, 100, 15], 2),          # the smallest K the tuned kernels take; four token tiles in one expert
    ],
)
def test_tq1_gemm_tiles(bp, act, E, N, K, counts, terms, tq1_gemm_kernel):
    got, want, kern = _run(bp, "tq1", E, N, K, counts, act, terms=terms, seed=K + N)
    assert kern == (tq1_gemm_kernel if act == "bf16" else "gemm_tq1_i8"), kern
    _check(got, want)


@pytest.mark.parametrize("K", [1024, 1280, 1536, 1792, 2048])  # K % 5 = 4, 0, 1, 2, 3: Kp = 205, 256, 308, 359, 410
@pytest.mark.parametrize("scale_dtype", [np.float16, "f32", "bf16"])
def test_tq1_gemm_over_converted_activations_reads_the_last_bytes_of_the_tensor(bp, tune, K, scale_dtype):
    """The last slice of the last row of the last expert ends at the tensor's last byte, or its 8-byte load one byte
    past it - and the hardware zeroes a dword that straddles the end of the buffer, valid bytes included, so that wave
    loads the window byte by byte. Every remainder of K / 5 (= every byte alignment of the rows); N = 48 leaves row tiles
    of the wave past N, N = 528 a second row block of 16 rows."""
    tune("BP_TUNE_TQ2G", "fp4")
    for E, N, counts in ((2, 48, [20, 33]), (2, 528, [1, 40])):
        got, want, kern = _run(bp, "tq1", E, N, K, counts, "bf16", seed=K, scale_dtype=scale_dtype)
        # (float32 scales: their ring does not fit in LDS beside the table and the transit area; the other kernel takes the call)
        assert kern == ("gemm_tq1_bf16" if scale_dtype == "f32" else "gemm_tq1f_bf16"), kern
        _check(got, want)


@pytest.mark.parametrize("ntok", [9, 16, 32])
def test_tq1_gemm_fp8_pieces_keep_small_activations(bp, ntok, tq1_gemm_kernel):
    """The grouped GEMM splits an activation into two E4M3 pieces under a power-of-two scale per block of 20: exact for
    bf16 values down to 2^-9 of the block's largest magnitude. Activations spread over 5 decades with outliers 1000 x
    the typical value must still come out far inside the general tolerance."""
    rng = np.random.default_rng(13)
    E, N, K = 2, 64, 4352
    packed, scales = synth_weights(13, E, N, K, GROUP, "tq1")
    T = E * ntok
    x = rng.standard_normal((T, K)).astype(np.float32) * np.exp(rng.uniform(-6, 6, (T, K))).astype(np.float32)
    x[:, ::97] *= 1000.0
    x = orc.bf16_round(x)
    want = np.zeros((T, N), np.float32)
    for e in range(E):
        c_gemm(x[e * ntok:(e + 1) * ntok], None, packed[0][e], scales[0][e].astype(np.float32), K, GROUP, "tq1", out=want[e * ntok:(e + 1) * ntok])
    got = bp.grouped_ternary_gemm(dev(x).to(torch.bfloat16), None, [0, ntok, 2 * ntok], [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq1").cpu().numpy()
    assert bp.ext().last_kernel() == tq1_gemm_kernel, bp.ext().last_kernel()
    assert rel_l2(got, want) <= 2e-4, rel_l2(got, want)
    z = np.zeros_like(x)  # all-zero activations: the block scale has nothing to go by
    got = bp.grouped_ternary_gemm(dev(z).to(torch.bfloat16), None, [0, ntok, 2 * ntok], [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq1")
    assert torch.equal(got, torch.zeros_like(got))


@pytest.mark.parametrize("ntok,chunk,want_kernel", [(2, False, "fp4_tq1_m2"), (2, True, "fp4_tq1_m2_cw"), (4, False, "fp4_tq1_m4"),
                                                    (6, False, "fp4_tq1_m6"), (8, False, "fp4_tq1_m8")])
def test_tq1_small_batches_fp8_pieces_keep_small_activations(bp, tune, ntok, chunk, want_kernel):
    """The small-batch variants (2 to 8 token rows per expert) keep two E4M3 pieces per activation under the group's
    power-of-two prescale: exact for bf16 values down to 2^-9 of the group's largest magnitude, at most 2^-17 of it
    dropped below. Activations spread over 5 decades with outliers 1000 x the typical value must still come out far
    inside the general tolerance, on the kernels that walk along their rows and on the one that streams them through LDS."""
    if chunk:
        tune("BP_TUNE_TQ1", "chunk")
    rng = np.random.default_rng(17 + ntok)
    E, N, K = 2, 272, 4352
    packed, scales = synth_weights(17, E, N, K, GROUP, "tq1")
    T = E * ntok
    x = rng.standard_normal((T, K)).astype(np.float32) * np.exp(rng.uniform(-6, 6, (T, K))).astype(np.float32)
    x[:, ::97] *= 1000.0
    x = orc.bf16_round(x)
    want = np.zeros((T, N), np.float32)
    for e in range(E):
        c_gemm(x[e * ntok:(e + 1) * ntok], None, packed[0][e], scales[0][e].astype(np.float32), K, GROUP, "tq1", out=want[e * ntok:(e + 1) * ntok])
    got = bp.grouped_ternary_gemm(dev(x).to(torch.bfloat16), None, [0, ntok, 2 * ntok], [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq1").cpu().numpy()
    kern = bp.ext().last_kernel()
    assert kern == want_kernel if chunk else kern.startswith(want_kernel) and not kern.endswith("_cw"), kern
    print("rel_l2", want_kernel, rel_l2(got, want))
    assert rel_l2(got, want) <= 2e-4, rel_l2(got, want)
    z = np.zeros_like(x)  # all-zero activations: the prescale has nothing to go by
    got = bp.grouped_ternary_gemm(dev(z).to(torch.bfloat16), None, [0, ntok, 2 * ntok], [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq1")
    assert torch.equal(got, torch.zeros_like(got))


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K", [1024, 2048, 5120, 7168])
@pytest.mark.parametrize("counts", [[2, 0, 1], [2, 2, 2], [4, 3, 1], [3, 0, 0], [8, 5, 1], [1, 6, 7], [5, 6, 0]])
def test_tq1_fp4_small_batches(bp, K, counts, act):
    """Up to 2, 4, 6, 8 token rows per expert: one operand tile per token (two fp8 pieces), one matrix instruction per
    token pair; experts with fewer rows than the launch's variant holds leave rows of the operand unused. Where the
    tiles of all of K do not fit in LDS (K = 5120 with 8 tokens, K = 7168 with 6 or 8) K is cut into segments, one
    launch each."""
    got, want, kern = _run(bp, "tq1", 3, 80, K, counts, act, terms=2, seed=K + 7 * sum(counts))
    m = max(counts)
    want_kernel = "fp4_tq1_m2" if m <= 2 else "fp4_tq1_m4" if m <= 4 else "fp4_tq1_m6" if m <= 6 else "fp4_tq1_m8"
    assert kern.startswith(want_kernel), kern
    _check(got, want)


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K,counts,last", [(2048, [9, 1, 0, 2, 1, 0, 12, 1], "fp4_tq1_m4"), (7168, [1, 16, 0, 3, 2, 1, 1, 5], "fp4_tq1_m8"),
                                           (4096, [2, 2, 10, 0, 0, 0, 1, 7], "fp4_tq1_m2"), (2048, [27, 0, 1, 0, 0, 0, 1, 3], "fp4_tq1_m4")])
def test_tq1_fp4_few_large_experts(bp, K, counts, last, act):
    """Up to 16 rows in a few experts while most have few (T <= 4 E): a launch for every expert's first 8 rows and one
    for the rest; experts with fewer rows than a launch's variant holds run the loop nest of their own pair count."""
    got, want, kern = _run(bp, "tq1", len(counts), 48, K, counts, act, terms=2, seed=K + 3)
    assert kern.startswith(last), kern
    _check(got, want)


def test_tq1_dense_batches_of_seven_or_eight_rows_run_on_the_tile_kernel_with_a_workspace(bp):
    """Seven or eight rows per expert, four or more on average, and at least 512 blocks of 512 output rows: the mirrored
    call brings a workspace and the call runs on the tile kernel over converted activations (one decode of the weights
    instead of two launches of the four-row kernel); six rows, few experts or int8 activations stay on the decode kernels."""
    from deepseekternarized_amd.kernels import _lib
    E, N, K = 128, 2048, 1024
    counts = [8] * (E - 3) + [7, 0, 5]
    T = sum(counts)
    lib = bp.ext().lib
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, T, N, K, E, 1, 8) > 0
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, T, N, K, E, 1, 7) > 0
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, T, N, K, E, 1, 6) == 0
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, 16 * 8, N, K, 16, 1, 8) == 0   # 64 blocks
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, 3 * E, N, K, E, 1, 8) == 0     # three rows per expert on average
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_I8, T, N, K, E, 1, 8) == 0
    got, want, kern = _run(bp, "tq1", E, N, K, counts, "bf16", seed=77)
    assert kern == "gemm_tq1f_bf16", kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", E, N, K, counts, "int8", seed=78)
    assert kern.startswith("fp4_tq1_m"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 16, N, K, [8] * 16, "bf16", seed=79)
    assert kern.startswith("fp4_tq1_m"), kern
    _check(got, want)


def test_tq1_fp4_upper_bound_max_rows(bp):
    """max_rows as an upper bound (64 for a decode step of 64 tokens) with offsets on the device: 8 launches of 8 rows,
    most of them without any row to take."""
    counts = [3, 0, 1, 11, 2, 0, 0, 1, 2, 5, 1, 1, 0, 2, 1, 1, 4, 0, 2, 1]
    got, want, kern = _run(bp, "tq1", len(counts), 48, 2048, counts, "bf16", terms=2, seed=31, max_rows=64)
    assert kern.startswith("fp4_tq1_m6"), kern  # (the bound is capped at the 38 rows of the call: 4 launches of 8 rows and one of 6)
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 3, 48, 2048, [30, 1, 2], "bf16", seed=32, max_rows=33)  # T > 4 E
    assert kern.startswith("gemm_tq1"), kern
    _check(got, want)


def test_tq1_small_batches_other_kernels(bp, tune):
    """fp16 activations (11 significant bits: more than two fp8 pieces hold) run as a pair of bf16 halves (8 + 3 bits) on
    the same kernel when the call brings a workspace (the mirrored call does); K that would take more than 4 segments
    goes to the kernels it went to before; the development switch keeps the multi-row MFMA kernel. K = 16384 with 4
    tokens runs as two segments of 13 chunks, with 8 tokens as four of 7 (the last one 5)."""
    got, want, kern = _run(bp, "tq1", 3, 80, 2048, [2, 4, 1], "f16", seed=21)
    assert kern.startswith("fp4_tq1_m4"), kern
    _check(got, want)
    assert rel_l2(got, want) <= 1e-5, rel_l2(got, want)  # (the halves are exact; what is left is the pieces' 2^-17)
    got, want, kern = _run(bp, "tq1", 2, 32, 16384, [4, 2], "bf16", seed=22)
    assert kern.startswith("fp4_tq1_m4"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 2, 32, 16384, [8, 3], "int8", seed=24)
    assert kern.startswith("fp4_tq1_m8"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq1", 2, 32, 20480, [7, 8], "bf16", seed=25)  # 32 chunks: 5 segments of 7
    assert not kern.startswith("fp4_tq1"), kern
    _check(got, want)
    tune("BP_TUNE_TQ1", "mfma")
    got, want, kern = _run(bp, "tq1", 3, 80, 2048, [2, 4, 1], "bf16", seed=23)
    assert kern.startswith("mfma_tq1"), kern
    _check(got, want)


def test_tq1_fp4_small_batches_misaligned_scales(bp):
    got, want, kern = _run(bp, "tq1", 2, 32, 2048, [3, 4], "bf16", seed=8, misalign_scales=True)
    assert kern.startswith("fp4_tq1_m4"), kern
    _check(got, want)


def test_tq1_mfma_scales_from_global_memory(bp, tune):
    got, want, kern = _run(bp, "tq1", 2, 32, 2048, [9, 4], "bf16", seed=8, misalign_scales=True)
    assert kern.startswith("gemm_tq1"), kern
    _check(got, want)
    tune("BP_TUNE_TQ1", "mfma")
    got, want, kern = _run(bp, "tq1", 2, 32, 2048, [9, 4], "bf16", seed=8, misalign_scales=True)
    assert kern.startswith("mfma_tq1") and kern.endswith("_gs"), kern
    _check(got, want)


# --------------------------------------------------------------------------- TQ2 decode GEMV with K split over the waves
# One token row per expert on the fp8 x fp4 matrix instruction (bp_tq2_gemv_fp4.hip; kernel names fp4_tq2_t1_ks and
# fp4_tq2_i8_t1_ks): the default for large single-token calls from K = 2048; BP_TUNE_TQ2V=k selects it wherever it can
# run, =n never.
@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("E,N,K,group,terms,sdt", [
    (3, 64, 1024, 128, 1, np.float16),      # 2 waves, a workgroup of one round
    (2, 144, 1280, 128, 2, "bf16"),         # an odd number of steps: the last wave's second step lies past the row
    (3, 1040, 4096, 256, 2, np.float16),    # a scale per 256 weights, stacked terms, 65 tiles (a last round of one tile)
    (2, 2064, 7168, 128, 1, np.float16),    # the headline K: 14 waves
    (1, 272, 8192, 128, 1, "bf16"),         # 16 waves
    (3, 528, 7168, 128, 2, "f32"),          # float32 scales (what the reference's wrappers pass): two 16-byte loads per wave and round
    (2, 272, 2304, 256, 1, "f32"),
    (5, 48, 768, 128, 1, np.float16),       # below the kernel's K: the other kernels
])
def test_tq2_single_token_gemv_with_k_split_over_the_waves(bp, tune, act, E, N, K, group, terms, sdt):
    tune("BP_TUNE_TQ2V", "k")
    counts = [1] * E
    if E > 2:
        counts[1] = 0  # an expert without a token row
    got, want, kern = _run(bp, "tq2", E, N, K, counts, act, terms=terms, seed=K + N, scale_dtype=sdt, group=group, max_rows=1)
    if K >= 1024:
        assert kern == ("fp4_tq2_i8_t1_ks" if act == "int8" else "fp4_tq2_t1_ks"), kern
    else:
        assert not kern.startswith("fp4_tq2"), kern
    _check(got, want)
    if act == "int8":  # fp8 pieces hold int8 values exactly and the sums are integers: only the order of the float32 scale products differs
        assert rel_l2(got, want) <= 1e-6, rel_l2(got, want)


def test_tq2_k_split_gemv_is_the_default_for_large_single_token_calls(bp):
    """64 experts x 64 row tiles at K = 2048 (16 tiles per CU): both activation dtypes take the kernel without a switch;
    the same call with two rows for one expert does not."""
    for act in ("bf16", "int8"):
        got, want, kern = _run(bp, "tq2", 64, 1024, 2048, [1] * 64, act, seed=5, max_rows=1)
        assert kern == ("fp4_tq2_i8_t1_ks" if act == "int8" else "fp4_tq2_t1_ks"), kern
        _check(got, want)
    got, want, kern = _run(bp, "tq2", 64, 1024, 2048, [1] * 63 + [2], "bf16", seed=6, max_rows=2)
    assert kern == "fp4_tq2_m2_ks", kern  # (a bound of two rows: the pair variant)
    _check(got, want)
    got, want, kern = _run(bp, "tq2", 64, 1024, 2048, [1] * 63 + [3], "bf16", seed=7, max_rows=3)
    assert kern == "fp4_tq2_m4_ks", kern  # (three or four rows: the variant for four)
    _check(got, want)
    got, want, kern = _run(bp, "tq2", 64, 1024, 2048, [1] * 63 + [5], "bf16", seed=8, max_rows=5)
    assert kern.startswith("mfma_tq2"), kern
    _check(got, want)


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("E,N,K,group,terms,sdt,counts", [
    (3, 272, 2048, 128, 1, np.float16, [2, 0, 1]),
    (2, 144, 1280, 128, 2, "bf16", [2, 2]),
    (3, 1040, 4096, 256, 2, np.float16, [1, 2, 2]),
    (2, 2064, 7168, 128, 1, np.float16, [2, 1]),
    (3, 528, 7168, 128, 2, "f32", [2, 2, 0]),
])
def test_tq2_token_pair_gemv_with_k_split_over_the_waves(bp, tune, act, E, N, K, group, terms, sdt, counts):
    """A pair of token rows per expert on the same kernel (two fp8 pieces per activation, rows 4 g + 2 t + p of operand A):
    experts with two rows, one row and none; stacked terms; scale types and group sizes."""
    if act == "int8" and sdt == "f32":
        pytest.skip("int8 activations with float32 scales stay on the other kernel")
    tune("BP_TUNE_TQ2V", "k")
    got, want, kern = _run(bp, "tq2", E, N, K, counts, act, terms=terms, seed=K + N + 1, scale_dtype=sdt, group=group, max_rows=2)
    assert kern == ("fp4_tq2_i8_m2_ks" if act == "int8" else "fp4_tq2_m2_ks"), kern
    _check(got, want)
    if act == "int8":
        assert rel_l2(got, want) <= 1e-6, rel_l2(got, want)


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("E,N,K,group,terms,sdt,counts", [
    (3, 272, 2048, 128, 1, np.float16, [4, 0, 3]),
    (2, 144, 2304, 128, 2, "bf16", [4, 1]),
    (3, 1040, 4096, 256, 2, np.float16, [2, 4, 3]),
    (2, 2064, 7168, 128, 1, np.float16, [4, 4]),
    (3, 528, 7168, 128, 2, "f32", [3, 4, 0]),
])
def test_tq2_four_token_gemv_with_k_split_over_the_waves(bp, tune, act, E, N, K, group, terms, sdt, counts):
    """Up to four token rows per expert on the same kernel: an accumulator tile per 64-byte step, rows 8 q + 2 t + p of
    operand A (the step's group q, token t, piece p); experts with four, three, two, one and no rows; stacked terms; an odd
    number of steps (the last wave's second step lies past the row)."""
    if act == "int8" and sdt == "f32":
        pytest.skip("int8 activations with float32 scales stay on the other kernel")
    tune("BP_TUNE_TQ2V", "k")
    got, want, kern = _run(bp, "tq2", E, N, K, counts, act, terms=terms, seed=K + N + 2, scale_dtype=sdt, group=group, max_rows=max(counts))
    assert kern == ("fp4_tq2_i8_m4_ks" if act == "int8" else "fp4_tq2_m4_ks"), kern
    _check(got, want)
    if act == "int8":
        assert rel_l2(got, want) <= 1e-6, rel_l2(got, want)


@pytest.mark.parametrize("fmt,N,rows,switch,off,want", [("tq2", 1536, 4, "BP_TUNE_TQ2V", "n", "fp4_tq2_m4_ks"), ("tq1", 3072, 4, "BP_TUNE_TQ1", "rows", "fp4_tq1_m4_cw")])
def test_decode_gemv_ranges_capped_by_lds_cover_every_row(bp, tune, fmt, N, rows, switch, off, want):
    """128 experts x 96 (192) row tiles at four token rows: a workgroup's LDS holds the sums of 32 (64) tiles, so an
    expert's tiles go to 4 workgroups of 24 (48) rather than 3 of 32 (64) - whole rounds of the resident workgroups. The
    launch is too large for the CPU kernel in a test's time: checked against the library's other kernel for these calls
    (each of them is checked against the CPU kernel at smaller sizes), on weights drawn on the device."""
    E, K = 128, 7168
    g = torch.Generator(device="cuda").manual_seed(N)
    packed = torch.empty(E, N, bp.packed_cols(fmt, K), dtype=torch.uint8, device="cuda")
    for e in range(E):
        packed[e] = bp.pack(torch.randint(-1, 2, (N, K), device="cuda", generator=g).to(torch.int8), fmt)
    scale = (0.02 * torch.randn(E, N, K // GROUP, device="cuda", generator=g).abs()).half()
    x = torch.randn(E * rows, K, device="cuda", generator=g).to(torch.bfloat16)
    offsets = [rows * e for e in range(E + 1)]
    got = bp.grouped_ternary_gemm(x, None, offsets, packed, scale, K, GROUP, fmt)
    assert bp.ext().last_kernel() == want, bp.ext().last_kernel()
    tune(switch, off)
    ref = bp.grouped_ternary_gemm(x, None, offsets, packed, scale, K, GROUP, fmt)
    assert bp.ext().last_kernel() != want
    got, ref = got.double(), ref.double()
    assert torch.isfinite(got).all()
    per_expert = ((got - ref).reshape(E, -1).norm(dim=1) / ref.reshape(E, -1).norm(dim=1)).max().item()
    assert per_expert <= REL_L2, per_expert
    per_tile = ((got - ref).reshape(E * rows, N // 16, 16).norm(dim=2) / ref.reshape(E * rows, N // 16, 16).norm(dim=2)).max().item()
    assert per_tile <= 10 * REL_L2, per_tile  # (no row tile left out or added twice)


def test_tq2_k_split_gemv_adds_to_the_output_and_keeps_other_rows(bp, tune):
    """The C-ABI call accumulates (include/bp_ternary.h): the kernel reads what it adds to when a workgroup starts and
    writes once at its end; rows of experts without a token and rows past N / 16 tiles of a workgroup stay as they were."""
    from deepseekternarized_amd.kernels import _lib
    tune("BP_TUNE_TQ2V", "k")
    lib = _lib.load()
    E, N, K = 3, 400, 2048
    packed, scales = synth_weights(3, E, N, K, GROUP, "tq2")
    rng = np.random.default_rng(3)
    x = orc.bf16_round(rng.standard_normal((2, K)).astype(np.float32))
    offsets = np.array([0, 1, 1, 2], np.int64)
    base = rng.standard_normal((2, N)).astype(np.float32)
    out = dev(base.copy())
    xd, pk, sc, od = dev(x).to(torch.bfloat16), dev(packed[0]), dev(scales[0]), dev(offsets)
    import ctypes
    pa = (ctypes.c_void_p * 1)(pk.data_ptr())
    sa = (ctypes.c_void_p * 1)(sc.data_ptr())
    rc = lib.bp_ternary_grouped_gemm(out.data_ptr(), xd.data_ptr(), _lib.BP_BF16, None, od.data_ptr(), None, pa, sa, _lib.BP_F16,
                                     1, 2, N, K, K // 4, K // GROUP, GROUP, E, _lib.BP_TQ2, 1, None, None)
    assert rc == 0, lib.bp_last_error()
    assert lib.bp_last_kernel().decode() == "fp4_tq2_t1_ks"
    want = base.copy()
    c_gemm(x[0:1], None, packed[0][0], scales[0][0].astype(np.float32), K, GROUP, "tq2", out=want[0:1])
    c_gemm(x[1:2], None, packed[0][2], scales[0][2].astype(np.float32), K, GROUP, "tq2", out=want[1:2])
    assert rel_l2(out.cpu().numpy(), want) <= 1e-5


def test_tq2_k_split_gemv_keeps_small_activations_next_to_outliers(bp, tune):
    """Three fp8 pieces under a power-of-two prescale per 128 activations represent bf16 values to 2^-20 of the group's
    largest magnitude; the matrix instruction's aligned sum of 128 products is what limits the result when a group
    holds values many decades apart: held to 5e-4 here (measured 1-2e-4; the general tolerance is 1e-3), and to 2e-5 on
    normally distributed activations (measured 1e-7 to 4e-6)."""
    tune("BP_TUNE_TQ2V", "k")
    rng = np.random.default_rng(21)
    E, N, K = 2, 64, 4096
    packed, scales = synth_weights(21, E, N, K, GROUP, "tq2")
    for spread, bound in ((0.0, 2e-5), (6.0, 5e-4)):
        x = rng.standard_normal((E, K)).astype(np.float32) * np.exp(rng.uniform(-spread, spread, (E, K))).astype(np.float32)
        if spread:
            x[:, ::97] *= 1000.0
        x = orc.bf16_round(x)
        want = np.zeros((E, N), np.float32)
        for e in range(E):
            c_gemm(x[e:e + 1], None, packed[0][e], scales[0][e].astype(np.float32), K, GROUP, "tq2", out=want[e:e + 1])
        got = bp.grouped_ternary_gemm(dev(x).to(torch.bfloat16), None, dev(np.array([0, 1, 2], np.int64)), [dev(packed[0])], [dev(scales[0])], K, GROUP, "tq2", max_rows=1).cpu().numpy()
        assert bp.ext().last_kernel() == "fp4_tq2_t1_ks"
        assert np.isfinite(got).all() and rel_l2(got, want) <= bound, (spread, rel_l2(got, want))


def test_tq2_k_split_gemv_replays_in_a_hip_graph(bp, tune):
    """The call captured into a HIP graph (the output's zero-fill is torch's fill kernel, the launch reads what it adds
    to and writes once): several replays with eager launches in between, every replay against the eager result."""
    tune("BP_TUNE_TQ2V", "k")
    E, N, K = 4, 528, 4096
    packed, scales = synth_weights(44, E, N, K, GROUP, "tq2", terms=2)
    rng = np.random.default_rng(44)
    pk, sc = [dev(p) for p in packed], [dev(s) for s in scales]
    off = dev(np.arange(E + 1, dtype=np.int64))
    x = dev(orc.bf16_round(rng.standard_normal((E, K)).astype(np.float32))).to(torch.bfloat16)
    want = bp.grouped_ternary_gemm(x, None, off, pk, sc, K, GROUP, "tq2", max_rows=1).clone()
    assert bp.ext().last_kernel() == "fp4_tq2_t1_ks"
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        bp.grouped_ternary_gemm(x, None, off, pk, sc, K, GROUP, "tq2", max_rows=1)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = bp.grouped_ternary_gemm(x, None, off, pk, sc, K, GROUP, "tq2", max_rows=1)
    for i in range(4):
        got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), i
        x2 = dev(orc.bf16_round(rng.standard_normal((E, K)).astype(np.float32))).to(torch.bfloat16)
        bp.grouped_ternary_gemm(x2, None, off, pk, sc, K, GROUP, "tq2", max_rows=1)  # eager work between the replays
        torch.cuda.synchronize()


def test_tq2_k_split_gemv_counts_the_unused_code_as_unpack_does(bp, tune):
    """pack never writes the 2-bit code 3. unpack reads it as +2 (boilerplate/ternary/pack.py:47-60: code - 1) and so does
    this kernel (E2M1 1.5 = 3 / 2, minus the offset); the reference's CPU kernel adds or subtracts by the trit's sign
    only (boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77), which makes such a weight +1 there."""
    tune("BP_TUNE_TQ2V", "k")
    rng = np.random.default_rng(8)
    E, N, K = 1, 32, 2048
    packed = rng.integers(0, 256, (E, N, K // 4), dtype=np.uint8)  # every code, 3 included
    scales = (rng.uniform(0.01, 0.1, (E, N, K // GROUP))).astype(np.float16)
    x = orc.bf16_round(rng.standard_normal((1, K)).astype(np.float32))
    trits = orc.unpack(packed[0], "tq2", K).astype(np.float64)
    assert trits.max() == 2
    sums = (trits.reshape(N, K // GROUP, GROUP) * x.astype(np.float64).reshape(1, K // GROUP, GROUP)).sum(-1)
    want = (sums * scales[0].astype(np.float64)).sum(-1)[None].astype(np.float32)
    got = bp.grouped_ternary_gemm(dev(x).to(torch.bfloat16), None, dev(np.array([0, 1], np.int64)), [dev(packed)], [dev(scales)], K, GROUP, "tq2", max_rows=1).cpu().numpy()
    assert bp.ext().last_kernel() == "fp4_tq2_t1_ks"
    assert rel_l2(got, want) <= 1e-5, rel_l2(got, want)


# --------------------------------------------------------------------------- TQ2 MFMA kernel
@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K,counts", [(1024, [1, 0, 1]), (2048, [1, 1, 1]), (7168, [3, 0, 16]), (4096, [33, 1, 20]), (32768, [1, 2, 0])])
def test_tq2_mfma_variants(bp, act, K, counts):
    """Single-token, 16-token and 32-token tiles; K = 32768 has more scales per row than the LDS tile takes."""
    got, want, kern = _run(bp, "tq2", 3, 2048 + 16 if K <= 2048 else 64, K, counts, act, terms=2 if K == 4096 else 1, seed=K + len(act))
    assert kern.startswith("gemm_tq2" if max(counts) > 16 else "mfma_tq2"), kern
    _check(got, want)


@pytest.mark.parametrize("rows", [3, 5, 7, 11])
def test_tq2_token_tiles_of_large_calls_stage_every_row(bp, tune, rows):
    """Large calls run the 16-wave variant of the token-tile kernel, whose activation tile holds 1.5 sixteen-element
    units per thread with 16-bit activations: with 3 - 7 or 9 - 11 rows per expert the tile is longer than one unit per
    thread, and every row of it has to be staged (the last rows once were not)."""
    tune("BP_TUNE_TQ2V", "n")  # (three rows: keep the K-split GEMV out of the way)
    E, N, K = 8, 4096, 4096
    got, want, kern = _run(bp, "tq2", E, N, K, [rows] * E, "bf16", seed=rows)
    assert kern == "mfma_tq2_bf16_r1_m1_w16", kern
    _check(got, want)
    for e in range(E):  # (the last row of each expert by itself: a tile's last rows are the ones that were left out)
        r = (e + 1) * rows - 1
        assert rel_l2(got[r], want[r]) <= REL_L2, (e, rel_l2(got[r], want[r]))


def test_tq2_bf16_scales_and_f32_scales(bp):
    got, want, kern = _run(bp, "tq2", 2, 64, 2048, [1, 9], "bf16", seed=11, scale_dtype=np.float32)
    assert kern.startswith("mfma_tq2"), kern
    _check(got, want)
    # float32 scales through the mirrored API
    packed, scales = synth_weights(12, 1, 64, 2048, GROUP, "tq2")
    x = orc.bf16_round(np.random.default_rng(12).standard_normal((5, 2048)).astype(np.float32))
    want = c_gemm(x, None, packed[0][0], scales[0][0].astype(np.float32), 2048, GROUP, "tq2")
    got = bp.ternary_gemm_float(dev(x).to(torch.bfloat16), dev(packed[0][0]), dev(scales[0][0]).float(), 2048, GROUP, "tq2")
    assert bp.ext().last_kernel().startswith("mfma_tq2")
    _check(got.cpu().numpy(), want)


# --------------------------------------------------------------------------- TQ2 grouped GEMM (token tiles of 32)
@pytest.fixture(params=["fp4", "bf16"])
def tq2_gemm_kernel(request, tune):
    """More than 16 rows per expert, bf16 activations: the fp8 x fp4 grouped GEMM over activations converted into a
    workspace (kernel name gemm_tq2f_bf16; BP_TUNE_TQ2G=fp4 runs it on shapes below its thresholds too) and the bf16
    MFMA kernel (gemm_tq2_bf16*; BP_TUNE_TQ2G=bf16). int8 activations run gemm_tq2_i8* either way."""
    tune("BP_TUNE_TQ2G", request.param)
    return "gemm_tq2f_" if request.param == "fp4" else "gemm_tq2_"


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize(
    "E,N,K,counts,terms",
    [
        (3, 64, 1024, [17, 0, 40], 2),        # the smallest K the tuned kernels take (four windows); two terms
        (5, 272, 2048, [32, 33, 1, 64, 16], 1),  # N not a multiple of a workgroup's rows; full, 1-row and 16-row tiles
        (11, 48, 3072, [20] * 11, 2),          # more experts than XCDs and not a multiple of 8; odd number of tiles
        (2, 528, 7168, [48, 31], 1),           # config-3 K; a second row block with 16 of its rows
        (3, 1040, 1280, [100, 9, 31], 1),      # an odd number of windows; three row blocks of the fp8 x fp4 kernel; four token tiles
    ],
)
def test_tq2_gemm_tiles(bp, act, E, N, K, counts, terms, tq2_gemm_kernel):
    got, want, kern = _run(bp, "tq2", E, N, K, counts, act, terms=terms, seed=K + N)
    assert kern.startswith(tq2_gemm_kernel if act == "bf16" else "gemm_tq2_i8"), kern
    _check(got, want)


def test_tq2_gemm_fp8_pieces_keep_small_activations(bp, tune):
    """Activations spread over five decades with 1000 x outliers: two E4M3 pieces under a scale per 32 activations."""
    tune("BP_TUNE_TQ2G", "fp4")
    rng = np.random.default_rng(77)
    E, N, K, counts = 2, 64, 2048, [33, 20]
    packed, scales = synth_weights(78, E, N, K, GROUP, "tq2")
    x = rng.standard_normal((sum(counts), K)).astype(np.float32) * np.exp(rng.uniform(-6, 6, (sum(counts), K))).astype(np.float32)
    x[rng.random(x.shape) < 0.01] *= 1000.0
    x = orc.bf16_round(x)
    offsets = np.concatenate([[0], np.cumsum(counts)])
    got = bp.grouped_ternary_gemm(dev(x).to(torch.bfloat16), None, dev(offsets), dev(packed[0]), dev(scales[0]), K, GROUP, "tq2", max_rows=max(counts))
    assert bp.ext().last_kernel().startswith("gemm_tq2f_"), bp.ext().last_kernel()
    want = np.concatenate([c_gemm(x[a:b], None, packed[0][e], scales[0][e].astype(np.float32), K, GROUP, "tq2")
                           for e, (a, b) in enumerate(zip(offsets[:-1], offsets[1:]))])
    rel = np.linalg.norm(got.cpu().numpy() - want) / np.linalg.norm(want)
    assert rel <= 1e-4, rel


@pytest.mark.parametrize("act", ["bf16", "int8"])
def test_tq2_gemm_float32_scales(bp, act, tq2_gemm_kernel):
    """What the reference's wrappers hand the kernel (`w_scale.float()`, boilerplate/kernels/ternary_cuda.py:95-97);
    also with one scale per 256 weights and an odd number of them per row."""
    got, want, kern = _run(bp, "tq2", 3, 80, 2304, [21, 0, 50], act, terms=2, seed=31, scale_dtype="f32")
    assert kern.startswith(tq2_gemm_kernel if act == "bf16" else "gemm_tq2_i8"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq2", 2, 528, 2304, [19, 33], act, terms=2, seed=32, scale_dtype="f32", group=256)
    assert kern.startswith(tq2_gemm_kernel if act == "bf16" else "gemm_tq2_i8"), kern
    _check(got, want)


def test_tq2_gemm_over_converted_activations_is_the_default_for_large_prefill(bp, tune):
    """Without a development switch: 8 experts x 800 rows x N = 2048 is above the thresholds; the result agrees with the bf16
    MFMA kernel's (which the tests above pin against the CPU restatement) to float32 summation order and the 2^-17 the
    fp8 pieces drop. The mirrored call brings the workspace; the plain C entry point (no workspace) keeps the bf16 kernel."""
    import ctypes as C

    from deepseekternarized_amd.kernels import _lib

    E, N, K, rows = 8, 2048, 1024, 800
    packed, scales = synth_weights(91, E, N, K, GROUP, "tq2", terms=2)
    pk, sc = [dev(p) for p in packed], [dev(s) for s in scales]
    g = torch.Generator(device="cuda").manual_seed(92)
    x = torch.randn(E * rows, K, device="cuda", generator=g).to(torch.bfloat16)
    offsets = torch.arange(0, E * rows + 1, rows, device="cuda", dtype=torch.int64)
    offsets[3] -= 13  # ragged tiles on both sides
    got = bp.grouped_ternary_gemm(x, None, offsets, pk, sc, K, GROUP, "tq2", max_rows=rows + 13)
    assert bp.ext().last_kernel() == "gemm_tq2f_bf16", bp.ext().last_kernel()
    lib = bp.ext().lib
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, E * rows, N, K, E, 2, rows + 13) > 0
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_I8, E * rows, N, K, E, 2, rows + 13) == 0
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, E * rows, N, K, E, 1, rows + 13) > 0  # (TQ1: the same kernel with the byte-table decode)
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, E * rows, N, K, E, 1, 8) == 0          # (the small-batch kernels take these)
    # a bound on the rows per expert so loose that most token tiles of the launch would not exist: no staged kernel, no workspace
    assert lib.bp_grouped_gemm_workspace_bytes(_lib.BP_BF16, E * rows, N, K, E, 2, E * rows) == 0
    tune("BP_TUNE_TQ2G", "bf16")
    want = bp.grouped_ternary_gemm(x, None, offsets, pk, sc, K, GROUP, "tq2", max_rows=rows + 13)
    assert bp.ext().last_kernel().startswith("gemm_tq2_bf16"), bp.ext().last_kernel()
    rel = ((got - want).norm() / want.norm()).item()
    assert rel <= 2e-5, rel
    tune("BP_TUNE_TQ2G", None)
    out = torch.zeros_like(got)
    pa = (C.c_void_p * 2)(*[p.data_ptr() for p in pk])
    sa = (C.c_void_p * 2)(*[s.data_ptr() for s in sc])
    args = (out.data_ptr(), x.data_ptr(), _lib.BP_BF16, None, offsets.data_ptr(), None, C.cast(pa, C.c_void_p), C.cast(sa, C.c_void_p),
            _lib.BP_F16, 2, E * rows, N, K, K // 4, K // GROUP, GROUP, E, 2, rows + 13)
    rc = lib.bp_ternary_grouped_gemm(*args, None, None)
    torch.cuda.synchronize()
    assert rc == 0 and lib.bp_last_kernel().decode().startswith("gemm_tq2_bf16")
    assert torch.equal(out, want)
    # a workspace that is too small: the same kernel as without one; a misaligned one: an error
    ws = torch.empty(4096, dtype=torch.uint8, device="cuda")
    out.zero_()
    rc = lib.bp_ternary_grouped_gemm_ws(*args, ws.data_ptr(), 4096, None)
    torch.cuda.synchronize()
    assert rc == 0 and lib.bp_last_kernel().decode().startswith("gemm_tq2_bf16") and torch.equal(out, want)
    rc = lib.bp_ternary_grouped_gemm_ws(*args, ws.data_ptr() + 8, 4096, None)
    assert rc != 0 and b"aligned" in lib.bp_last_error()


def test_tq2_gemm_scales_from_global_memory_and_other_scale_dtypes(bp, tq2_gemm_kernel):
    """K = 10240: 256 rows x 80 groups of scales do not fit beside the bf16 kernel's two activation tiles; bf16 scales; float32 scales."""
    got, want, kern = _run(bp, "tq2", 2, 64, 10240, [33, 18], "bf16", seed=21)
    assert kern == ("gemm_tq2_bf16_gs" if tq2_gemm_kernel == "gemm_tq2_" else "gemm_tq2f_bf16"), kern
    _check(got, want)
    got, want, kern = _run(bp, "tq2", 2, 64, 2048, [18, 40], "bf16", seed=22, scale_dtype=np.float32)  # bf16 scales
    assert kern.startswith(tq2_gemm_kernel), kern
    _check(got, want)
    packed, scales = synth_weights(23, 1, 80, 2048, GROUP, "tq2")
    x = orc.bf16_round(np.random.default_rng(23).standard_normal((137, 2048)).astype(np.float32))
    want = c_gemm(x, None, packed[0][0], scales[0][0].astype(np.float32), 2048, GROUP, "tq2")
    got = bp.ternary_gemm_float(dev(x).to(torch.bfloat16), dev(packed[0][0]), dev(scales[0][0]).float(), 2048, GROUP, "tq2")
    assert bp.ext().last_kernel().startswith("gemm_tq2")
    _check(got.cpu().numpy(), want)


@pytest.mark.parametrize("fmt,prefix", [("tq1", "mfma_tq1"), ("tq2", "mfma_tq2")])
def test_one_dense_linear_on_a_decode_batch_takes_the_16_token_tiles(bp, fmt, prefix):
    """A single linear (E = 1) with a few dozen rows: the 32-token-tile kernels would launch a handful of workgroups, so the
    call goes to the 16-token tiles (same contract, more workgroups)."""
    packed, scales = synth_weights(29, 1, 272, 2048, GROUP, fmt)
    x = orc.bf16_round(np.random.default_rng(29).standard_normal((64, 2048)).astype(np.float32))
    want = c_gemm(x, None, packed[0][0], scales[0][0].astype(np.float32), 2048, GROUP, fmt)
    got = bp.ternary_gemm_float(dev(x).to(torch.bfloat16), dev(packed[0][0]), dev(scales[0][0]), 2048, GROUP, fmt)
    assert bp.ext().last_kernel().startswith(prefix), bp.ext().last_kernel()
    _check(got.cpu().numpy(), want)


# --------------------------------------------------------------------------- float32 scales (TQ1)
@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K,counts,prefix", [(2048, [1, 0, 1], "fp4_tq1"), (7168, [1, 1, 1], "fp4_tq1"), (2048, [3, 16, 1], "gemm_tq1"),
                                              (7168, [20, 2, 9], "gemm_tq1"), (2048, [2, 1, 0], "fp4_tq1_m2"), (7168, [3, 4, 1], "fp4_tq1_m4"),
                                              (7168, [7, 0, 5], "fp4_tq1_m8"), (2304, [12, 0, 0], "fp4_tq1_m4")])
def test_tq1_float32_scales(bp, act, K, counts, prefix):
    """boilerplate/kernels/ternary_cuda.py:95-97 hands the kernel `w_scale.float()`: the tuned TQ1 kernels take it."""
    got, want, kern = _run(bp, "tq1", 3, 272, K, counts, act, terms=2, seed=K + len(act), scale_dtype="f32")
    assert kern.startswith(prefix), kern
    _check(got, want)


# --------------------------------------------------------------------------- TQ2 with K % 1024 != 0 (whole 256-trit steps)
@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K", [1280, 2304, 11008])
@pytest.mark.parametrize("counts,prefix", [([1, 1, 0], "mfma_tq2"), ([16, 0, 5], "mfma_tq2"), ([33, 2, 17], "gemm_tq2")])
def test_tq2_partial_last_block(bp, act, K, counts, prefix):
    """The last block of four steps (and the last activation tile) is partial; scale rows are not 16-byte multiples."""
    got, want, kern = _run(bp, "tq2", 3, 48, K, counts, act, terms=2 if K == 2304 else 1, seed=K + sum(counts))
    assert kern.startswith(prefix), kern
    _check(got, want)


def test_device_offsets_with_row_bound(bp):
    """Device offsets: the launch covers `max_rows` rows per expert; the exact widest count gives the host-offset result."""
    rng = np.random.default_rng(31)
    E, N, K, counts = 5, 64, 2048, [40, 0, 3, 17, 33]
    packed, scales = synth_weights(31, E, N, K, GROUP, "tq2")
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    x = dev(orc.bf16_round(rng.standard_normal((int(offsets[-1]), K)).astype(np.float32))).to(torch.bfloat16)
    pk, sc = [dev(p) for p in packed], [dev(s) for s in scales]
    want = bp.grouped_ternary_gemm(x, None, offsets.tolist(), pk, sc, K, GROUP, "tq2")
    got = bp.grouped_ternary_gemm(x, None, dev(offsets), pk, sc, K, GROUP, "tq2", max_rows=max(counts))
    assert torch.equal(got, want)
    loose = bp.grouped_ternary_gemm(x, None, dev(offsets), pk, sc, K, GROUP, "tq2")  # default bound: all rows
    assert torch.equal(loose, want)


@pytest.mark.parametrize("fmt,act,tokens", [("tq1", "bf16", 1), ("tq2", "int8", 5), ("tq2", "bf16", 40)])
def test_moe_layer_graph_replays_match_eager(bp, fmt, act, tokens):
    """The captured layer against the eager one, on several replays with different inputs and eager work in between."""
    from deepseekternarized_amd.moe import TernaryMoE

    H, I, E, k = 1024, 256, 8, 2
    stacks = []
    for (N, K), seed in (((I, H), 41), ((I, H), 42), ((H, I), 43)):
        packed, scales = synth_weights(seed, E, N, K, GROUP, fmt, terms=2)
        stacks.append([(dev(p), dev(s)) for p, s in zip(packed, scales)])
    moe = TernaryMoE(*stacks, hidden=H, inter=I, top_k=k, fmt=fmt, group=GROUP, act=act)
    run = moe.graphed(tokens)
    g = torch.Generator(device="cuda").manual_seed(44)
    for rep in range(4):
        x = torch.randn(tokens, H, device="cuda", generator=g).to(torch.bfloat16)
        logits = torch.randn(tokens, E, device="cuda", generator=g)
        want = moe(x, logits).clone()  # eager launches between the replays
        torch.cuda.synchronize()
        got = run(x, logits).clone()
        torch.cuda.synchronize()
        assert torch.isfinite(got).all() and torch.equal(got, want), (rep, (got.float() - want.float()).abs().max().item())
    with pytest.raises(ValueError):
        moe.graphed(0)


# --------------------------------------------------------------------------- scale groups of 256
@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("fmt,K,counts,prefix", [
    ("tq2", 2048, [1, 0, 1], "mfma_tq2"), ("tq2", 7168, [16, 2, 5], "mfma_tq2"), ("tq2", 3072, [40, 1, 20], "gemm_tq2"),
    ("tq1", 2048, [1, 1, 0], "fp4_tq1"), ("tq1", 7168, [1, 0, 1], "fp4_tq1"), ("tq1", 7168, [9, 16, 2], "gemm_tq1"),
    ("tq1", 2560, [3, 0, 20], "gemm_tq1"), ("tq1", 2048, [2, 2, 1], "fp4_tq1_m2"), ("tq1", 7168, [4, 0, 3], "fp4_tq1_m4"),
    ("tq1", 7168, [1, 6, 5], "fp4_tq1_m6"), ("tq1", 2560, [1, 0, 11], "fp4_tq1_m4"),
])
def test_group_256(bp, act, fmt, K, counts, prefix):
    """configs/policy/std_absmean_tq{1,2}_g256.yaml: one scale per 256 weights; the tuned kernels treat it as two 128-wide groups."""
    got, want, kern = _run(bp, fmt, 3, 272, K, counts, act, terms=2, seed=K + sum(counts), group=256)
    assert kern.startswith(prefix), kern
    _check(got, want)


# --------------------------------------------------------------------------- activations that are not finite
@pytest.mark.parametrize("fmt,counts,prefix", [
    ("tq1", [1, 1], "fp4_tq1_t1"), ("tq1", [1, 1], "fp4_tq1_t1_cw"), ("tq1", [2, 2], "fp4_tq1_m2_cw"), ("tq1", [4, 3], "fp4_tq1_m4"), ("tq1", [20, 12], "gemm_tq1"),
    ("tq2", [1, 1], "mfma_tq2"), ("tq2", [1, 1], "fp4_tq2_t1_ks"), ("tq2", [9, 16], "mfma_tq2"), ("tq2", [40, 33], "gemm_tq2_"), ("tq2", [40, 33], "gemm_tq2f_"),
])
def test_non_finite_activations_never_give_finite_wrong_values(bp, tune, fmt, counts, prefix):
    """The reference's CPU kernel skips zero weights (boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77), so a NaN or an
    infinite activation makes exactly the outputs with a nonzero weight at that k non-finite. The tuned kernels multiply
    zeros too (0 x Inf = NaN) or scale whole blocks: they may make more outputs of that token non-finite, but every
    output the reference makes non-finite must be non-finite here, and tokens without such an activation are untouched."""
    E, N, K = 2, 64, 2048
    if prefix == "gemm_tq2f_":
        tune("BP_TUNE_TQ2G", "fp4")
    if prefix.endswith("_cw"):
        tune("BP_TUNE_TQ1", "chunk")
    if prefix.startswith("fp4_tq2"):
        tune("BP_TUNE_TQ2V", "k")
    rng = np.random.default_rng(5)
    packed, scales = synth_weights(17, E, N, K, GROUP, fmt)
    trits = np.stack([orc.unpack(packed[0][e], fmt, K) for e in range(E)])
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    T = int(offsets[-1])
    x = orc.bf16_round(rng.standard_normal((T, K)).astype(np.float32))
    bad_tok = [0, T - 1]  # the first token of expert 0 gets a NaN, the last token of expert 1 an infinity
    x[0, 777] = np.nan
    x[T - 1, 130] = np.inf
    got = bp.grouped_ternary_gemm(dev(x).to(torch.bfloat16), None, offsets.tolist(), [dev(packed[0])], [dev(scales[0])], K, GROUP, fmt).cpu().numpy()
    assert bp.ext().last_kernel().startswith(prefix), bp.ext().last_kernel()
    assert not np.isfinite(got[0, trits[0][:, 777] != 0]).any()
    assert not np.isfinite(got[T - 1, trits[1][:, 130] != 0]).any()
    clean = np.setdiff1d(np.arange(T), bad_tok)
    if clean.size:
        want = np.zeros((T, N), np.float32)
        for e in range(E):
            a, b = int(offsets[e]), int(offsets[e + 1])
            c_gemm(np.nan_to_num(x[a:b], nan=0.0, posinf=0.0), None, packed[0][e], scales[0][e].astype(np.float32), K, GROUP, fmt, out=want[a:b])
        assert np.isfinite(got[clean]).all()
        assert rel_l2(got[clean], want[clean]) <= REL_L2
    # the reference-order kernel skips zero weights exactly like the reference
    ref = bp.grouped_ternary_gemm(dev(x), None, offsets.tolist(), [dev(packed[0])], [dev(scales[0])], K, GROUP, fmt, backend="torch").cpu().numpy()
    assert np.array_equal(~np.isfinite(ref[0]), trits[0][:, 777] != 0)
    assert np.array_equal(~np.isfinite(ref[T - 1]), trits[1][:, 130] != 0)


# --------------------------------------------------------------------------- float32 / fp16 activations beyond the single-token TQ1 kernels
@pytest.mark.parametrize("act", ["f32", "f16"])
@pytest.mark.parametrize("fmt,M", [("tq2", 1), ("tq2", 8), ("tq1", 8), ("tq2", 40)])
def test_float_activations_run_on_the_bf16_kernels_as_a_pair(bp, fmt, M, act):
    """Config 0's inputs (TQ2, K = 4096, N = 2048, M in {1, 8}, float32 activations; the reference runs them on its CPU
    kernel's float path, boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77, 114-124) and their fp16 / TQ1 / prefill
    relatives: split into hi + lo bf16 halves and multiplied by the bf16 kernels, both products added into the output.
    Held to the reference's own float-path tolerance (tests/test_ternary.py:98: rtol 1e-4, atol 1e-3)."""
    N, K = 2048, 4096
    rng = np.random.default_rng(M)
    packed, scales = synth_weights(5, 1, N, K, GROUP, fmt)
    x = rng.standard_normal((M, K)).astype(np.float32)
    if act == "f16":
        x = x.astype(np.float16).astype(np.float32)
    xd = dev(x).half() if act == "f16" else dev(x)
    got = bp.ternary_gemm_float(xd, dev(packed[0][0]), dev(scales[0][0]), K, GROUP, fmt)
    kern = bp.ext().last_kernel()
    assert kern.startswith(("mfma_" + fmt, "gemm_" + fmt, "fp4_" + fmt)) and "general" not in kern, kern
    want = c_gemm(x, None, packed[0][0], scales[0][0].astype(np.float32), K, GROUP, fmt)
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-4, atol=1e-3)
    # without a workspace (the plain C entry point): the general kernel, same numbers
    out = torch.zeros(M, N, device="cuda")
    offs = torch.tensor([0, M], device="cuda")
    bp.ext().lib.bp_set_kernel_policy(0)
    import ctypes as C
    from deepseekternarized_amd.kernels import _lib
    pk, sc = dev(packed[0]), dev(scales[0])
    pa, sa = (C.c_void_p * 1)(pk.data_ptr()), (C.c_void_p * 1)(sc.data_ptr())
    rc = bp.ext().lib.bp_ternary_grouped_gemm(out.data_ptr(), xd.data_ptr(), _lib.dtype_code(xd.dtype), None, offs.data_ptr(), None, C.cast(pa, C.c_void_p),
                                              C.cast(sa, C.c_void_p), _lib.BP_F16, 1, M, N, K, packed[0].shape[-1], K // GROUP, GROUP, 1, 2 if fmt == "tq2" else 1, M, None, None)
    torch.cuda.synchronize()
    assert rc == 0 and bp.ext().last_kernel().startswith("general"), bp.ext().last_kernel()
    np.testing.assert_allclose(out.cpu().numpy(), want, rtol=1e-4, atol=1e-3)


# --------------------------------------------------------------------------- packed tensors that start at any byte
@pytest.mark.parametrize("counts,act,switch,prefix", [
    ([1, 1], "bf16", None, "fp4_tq1_t1_ks"), ([1, 1], "int8", None, "fp4_tq1_t1_ks"), ([3, 2], "bf16", None, "fp4_tq1_m4"),
    ([1, 1], "bf16", ("BP_TUNE_TQ1", "chunk"), "fp4_tq1_t1_cw"), ([2, 1], "bf16", ("BP_TUNE_TQ1", "chunk"), "fp4_tq1_m2_cw"),
    ([1, 1], "bf16", ("BP_TUNE_TQ1", "lut"), "lut_tq1"), ([12, 3], "bf16", ("BP_TUNE_TQ1", "mfma"), "mfma_tq1"),
    ([9, 20], "bf16", None, "gemm_tq1f"), ([9, 20], "bf16", ("BP_TUNE_TQ2G", "bf16"), "gemm_tq1_"), ([9, 20], "int8", None, "gemm_tq1_"),
])
@pytest.mark.parametrize("K", [2048, 1280])  # Kp = 410, and 256: whole chunks of 128 bytes, so a row at an odd address ends in the chunk after its last
def test_tq1_packed_tensor_at_every_byte_alignment(bp, tune, counts, act, switch, prefix, K):
    """TQ1 rows start at any byte, and so may the tensor: a view 1, 2 or 3 bytes into an allocation, with other bytes
    behind it. The kernels read the rows through a buffer whose base is aligned down to a dword; its range has to end
    with the dword that holds the tensor's last byte (a dword that straddles the end of a range reads as zero, and the
    last row's last bytes with it). Every offset gives the bits of offset 0."""
    if switch:
        tune(*switch)
    E, N = len(counts), 48 if "cw" not in prefix else 2064
    rng = np.random.default_rng(5)
    packed, scales = synth_weights(5, E, N, K, GROUP, "tq1", terms=1)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    T = int(offsets[-1])
    x, xs, xd, xsd = _activations(rng, T, K, act)
    want = np.zeros((T, N), np.float32)
    for e in range(E):
        a, b = int(offsets[e]), int(offsets[e + 1])
        c_gemm(x[a:b], None if xs is None else xs[a:b], packed[0][e], scales[0][e].astype(np.float32), K, GROUP, "tq1", out=want[a:b])
    p, first = packed[0], None
    for off in (0, 1, 2, 3):
        buf = torch.full((p.size + 64,), 77, dtype=torch.uint8, device="cuda")  # (what lies behind the tensor must not matter)
        base = (16 - buf.data_ptr() % 16) % 16 + off
        buf[base:base + p.size] = dev(p).reshape(-1)
        view = buf[base:base + p.size].view(p.shape)
        assert view.data_ptr() % 4 == off
        got = bp.grouped_ternary_gemm(xd, xsd, offsets.tolist(), [view], [dev(scales[0])], K, GROUP, "tq1").cpu().numpy()
        assert bp.ext().last_kernel().startswith(prefix), bp.ext().last_kernel()
        _check(got, want)
        first = got if first is None else first
        assert np.array_equal(got, first), off


@pytest.mark.parametrize("act", ["bf16", "int8"])
@pytest.mark.parametrize("K,counts", [(2304, [8]), (5376, [1, 0, 1]), (4352, [1, 24]), (9472, [2])])
@pytest.mark.parametrize("scale_dtype", [np.float16, "f32"])
def test_tq2_group_256_with_an_odd_number_of_scales_per_row(bp, act, K, counts, scale_dtype):
    """K / 256 odd with one scale per 256 weights: every other row of 2-byte scales starts in the middle of a dword. The
    tuned TQ2 kernels read a row's scales in dword-aligned pieces and leave such calls to the general kernel (float32
    scales keep their rows aligned and stay on the tuned kernels)."""
    got, want, kern = _run(bp, "tq2", len(counts), 144, K, counts, act, seed=K, scale_dtype=scale_dtype, group=256)
    assert kern.startswith("general") == (scale_dtype is np.float16), kern
    _check(got, want)

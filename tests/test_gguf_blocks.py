"""llama.cpp TQ1_0 / TQ2_0 blocks from single-term ternary weights and back (boilerplate/format/gguf_export.py:45-58,
103-114; the reference's acceptance test tests/test_gguf_export.py:54-75: the blocks dequantize to unpack x scale, bit
for bit). The `gguf` package the reference calls is absent here: the oracle restates llama.cpp's published block layout
(oracle/ternary_oracle.py, "ggml TQ1_0 / TQ2_0 blocks") and is pinned by blocks worked out by hand from those formulas."""

import numpy as np
import pytest
import torch

from _util import orc, synth_trits

QK = 256


def _weight(seed, N, K):
    rng = np.random.default_rng(seed)
    trits = synth_trits(rng, (N, K))
    scale = (0.02 * np.abs(rng.standard_normal((N, K // QK)))).astype(np.float16)
    trits[0, :QK] = 0          # an all-zero block: d = 0, every digit 1
    if N > 1:
        scale[1, 0] = 0        # a zero scale under nonzero trits: the values are 0, so is d
    return trits, scale


def test_oracle_blocks_worked_by_hand():
    """TQ2_0: weight j of a chunk of 128 sits in byte j % 32 at bits 2 (j / 32). TQ1_0: byte = ceil(256 q / 243),
    q = sum digit 3^(4 - n), first weight most significant."""
    v = np.zeros((1, QK), np.float32)
    v[0, 0], v[0, 33], v[0, 128 + 96 + 5] = 0.5, -0.5, 0.5   # digits 2, 0, 2; everything else 1
    b = orc.gguf_quantize(v, "tq2_0")[0]
    assert b.size == 66
    ones = 0b01010101
    assert b[0] == (ones & ~0b11) | 0b10            # weight 0: byte 0, bits 0-1 = 2
    assert b[1] == (ones & ~0b1100) | 0b0000        # weight 33 = 1 + 32: byte 1, bits 2-3 = 0
    assert b[32 + 5] == (ones & ~0b11000000) | 0b10000000   # chunk 1, weight 96 + 5: byte 5 of the chunk, bits 6-7 = 2
    assert all(x == ones for i, x in enumerate(b[:64]) if i not in (0, 1, 37))
    assert b[64:].view(np.float16)[0] == np.float16(0.5)
    # TQ1_0: all digits 1 -> q = 121 -> ceil(121 * 256 / 243) = 128; qh: q = 40 * 3 = 120 -> ceil(120 * 256 / 243) = 127
    z = orc.gguf_quantize(np.zeros((1, QK), np.float32), "tq1_0")[0]
    assert z.size == 54 and (z[:48] == 128).all() and (z[48:52] == 127).all() and (z[52:] == 0).all()
    p = orc.gguf_quantize(np.full((1, QK), 0.25, np.float32), "tq1_0")[0]   # all +1: q = 242 -> 255; qh: 80 * 3 = 240 -> ceil(252.8) = 253
    assert (p[:48] == 255).all() and (p[48:52] == 253).all() and p[52:].view(np.float16)[0] == np.float16(0.25)
    m = orc.gguf_quantize(np.full((1, QK), -0.25, np.float32), "tq1_0")[0]  # all -1: q = 0
    assert (m[:52] == 0).all()
    v = np.zeros((1, QK), np.float32)
    v[0, 0], v[0, 32], v[0, 160 + 16 * 4 + 3], v[0, 240 + 2 + 4 * 3] = 1.0, -1.0, 1.0, -1.0
    b = orc.gguf_quantize(v, "tq1_0")[0]
    assert b[0] == -(-(2 * 81 + 0 * 27 + 9 + 3 + 1) * 256 // 243)          # byte 0: digits 2 (weight 0), 0 (weight 32), 1, 1, 1
    assert b[32 + 3] == -(-(81 + 27 + 9 + 3 + 2) * 256 // 243)             # byte 35: its last digit (n = 4) is weight 160 + 3 + 64
    assert b[48 + 2] == -(-((27 + 9 + 3 + 0) * 3) * 256 // 243)            # qh[2]: its last digit (n = 3) is weight 240 + 2 + 12
    # every byte value the encoder can produce decodes to the digits it was made from
    for q in range(243):
        byte = (q * 256 + 242) // 243
        assert byte < 256
        digits = [(((byte * 3 ** n) & 0xFF) * 3) >> 8 for n in range(5)]
        assert sum(d * 3 ** (4 - n) for n, d in enumerate(digits)) == q


@pytest.mark.parametrize("qtype", ["tq1_0", "tq2_0"])
def test_oracle_round_trip_is_exact(qtype):
    """The check the reference makes on every converted tensor (gguf_export.py:109-113)."""
    trits, scale = _weight(3, 6, 1024)
    values = trits.astype(np.float32) * np.repeat(scale.astype(np.float32), QK, 1)
    blocks = orc.gguf_quantize(values, qtype)
    assert blocks.shape == (6, 4 * (54 if qtype == "tq1_0" else 66))
    assert np.array_equal(orc.gguf_dequantize(blocks, qtype, 1024), values)
    with pytest.raises(ValueError):
        orc.gguf_quantize(values[:, :300], qtype)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("qtype", ["tq1", "tq2"])
def test_device_blocks_equal_the_oracle_and_round_trip(fmt, qtype):
    import deepseekternarized_amd as bp
    from deepseekternarized_amd.gguf_blocks import from_gguf_blocks, to_gguf_blocks

    N, K = 40, 2304
    trits, scale = _weight(7, N, K)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    term = bp.PackedTerm(bp.pack(dev(trits), fmt), dev(scale))
    blocks = to_gguf_blocks(term, K, fmt, 256, qtype)
    values = trits.astype(np.float32) * np.repeat(scale.astype(np.float32), QK, 1)
    want = orc.gguf_quantize(values, qtype + "_0")
    assert np.array_equal(blocks.cpu().numpy(), want)
    # the reference's acceptance check: the blocks dequantize to unpack x scale, bit for bit
    assert np.array_equal(orc.gguf_dequantize(blocks.cpu().numpy(), qtype + "_0", K), values)
    # ... and back into either packing: the same values again
    for fmt2 in ("tq1", "tq2"):
        back = from_gguf_blocks(blocks, K, fmt2, qtype)
        got = bp.unpack(back.packed, fmt2, K).float().cpu().numpy() * np.repeat(back.scale.float().cpu().numpy(), QK, 1)
        assert np.array_equal(got, values)
    with pytest.raises(ValueError, match="group 128"):
        to_gguf_blocks(term, K, fmt, 128, qtype)
    with pytest.raises(ValueError, match="fp16"):
        to_gguf_blocks(bp.PackedTerm(term.packed, term.scale.to(torch.bfloat16)), K, fmt, 256, qtype)
    with pytest.raises(ValueError, match="multiple of 256"):
        to_gguf_blocks(term, K - 128, fmt, 256, qtype)

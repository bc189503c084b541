"""Mode B's device decoder (bp_huff_decode; reference: boilerplate/kernels/csrc/huffman_cuda_kernel.cu:12-79,
boilerplate/format/entropy.py) against the oracle, which is pinned to the reference's own code lengths and compiled
encoder / decoder (tests/golden/huffman_ref.npz, written by tests/golden/make_huffman_fixture.py; live against
oracle/_ref where that build exists)."""

from pathlib import Path

import numpy as np
import pytest
import torch

from _util import reference_build
from oracle import huffman_oracle as H

GOLDEN = Path(__file__).resolve().parent / "golden" / "huffman_ref.npz"


def _cases():
    z = np.load(GOLDEN, allow_pickle=False)
    names = sorted({k.split(".")[0] for k in z.files})
    return {n: {k.split(".", 1)[1]: z[k] for k in z.files if k.startswith(n + ".")} for n in names}


def test_oracle_against_the_reference_fixture():
    """Code lengths (heap tie-breaking included), canonical codes, stream bytes and offsets equal the reference's."""
    for name, c in _cases().items():
        sym, block = c["sym"], int(c["block"][0])
        lens = H.code_lengths(np.bincount(sym, minlength=256))
        assert np.array_equal(lens, c["lens"]), name
        codes = H.canonical_codes(lens)
        assert np.array_equal(codes, c["codes"]), name
        stream, offsets = H.huff_encode(sym, codes, lens, block)
        assert np.array_equal(stream, c["stream"]) and np.array_equal(offsets, c["offsets"]), name
        assert np.array_equal(H.huff_decode(stream, offsets, sym.size, block, H.decode_table(lens), 12), sym), name
    assert _cases()["skewed"]["lens"].max() == 12  # the length limit binds in that case
    assert _cases()["one_symbol"]["lens"][7] == 1


def test_oracle_hand_worked_stream():
    """Three symbols with counts 5, 2, 1: lengths 1, 2, 2; canonical codes 0, 10, 11; 'abacab..' written MSB first."""
    freq = np.zeros(256, np.int64)
    freq[[10, 20, 30]] = (5, 2, 1)
    lens = H.code_lengths(freq)
    assert lens[[10, 20, 30]].tolist() == [1, 2, 2]
    codes = H.canonical_codes(lens)
    assert codes[[10, 20, 30]].tolist() == [0b0, 0b10, 0b11]
    sym = np.array([10, 20, 10, 30, 10, 20, 10, 10], np.uint8)  # 0 10 0 11 0 10 0 0 -> 0100 1101 000.....
    stream, offsets = H.huff_encode(sym, codes, lens, 3)
    assert stream[:2].tolist() == [0b01001101, 0b00000000] and stream.size == 2 + 8
    assert offsets.tolist() == [0, 4, 9, 11]  # blocks of 3 symbols: 4 bits, 5 bits, 2 bits
    lut = H.decode_table(lens, 4)
    assert lut[0] == (10 << 8) | 1 and lut[0b1000] == (20 << 8) | 2 and lut[0b1111] == (30 << 8) | 2
    assert np.array_equal(H.huff_decode(stream, offsets, 8, 3, lut, 4), sym)
    with pytest.raises(ValueError):
        H.huff_decode(stream, [0, 4, 9, 12], 8, 3, lut, 4)       # a block that does not end on its end bit
    with pytest.raises(ValueError):
        H.canonical_codes(np.array([1, 1, 1] + [0] * 253, np.uint8))  # oversubscribed


def test_oracle_against_the_reference_build_live():
    ext = reference_build()
    if ext is None:
        pytest.skip("oracle/_ref is not built on this machine")
    rng = np.random.default_rng(3)
    sym = rng.choice(200, size=30000, p=np.random.default_rng(4).dirichlet(np.ones(200) * 0.3)).astype(np.uint8)
    lens = H.code_lengths(np.bincount(sym, minlength=256))
    codes = H.canonical_codes(lens)
    stream, offsets = H.huff_encode(sym, codes, lens, 4096)
    rs, ro = ext.huff_encode(torch.from_numpy(sym), torch.from_numpy(codes), torch.from_numpy(lens), 4096)
    assert np.array_equal(stream, rs.numpy()) and np.array_equal(offsets, ro.numpy())
    back = ext.huff_decode(rs, ro, sym.size, 4096, torch.from_numpy(H.decode_table(lens)), 12)
    assert np.array_equal(back.numpy(), sym)


def test_host_tables_equal_the_oracle():
    from deepseekternarized_amd import entropy

    c = _cases()["skewed"]
    lens = torch.from_numpy(c["lens"])
    assert np.array_equal(entropy.canonical_codes(lens).numpy(), c["codes"])
    assert np.array_equal(entropy.decode_table(lens, 12).numpy(), H.decode_table(c["lens"], 12))
    with pytest.raises(ValueError):
        entropy.decode_table(lens, 8)
    with pytest.raises(ValueError):
        entropy.decode({"stream": torch.zeros(2, dtype=torch.uint8), "offsets": torch.zeros(2, dtype=torch.int64), "lens": lens}, 5)


@pytest.mark.gpu
def test_device_decode_of_the_reference_streams():
    """The streams the reference's encoder wrote, decoded on the device: 1-byte symbols, and 2-byte elements with the raw
    low bytes interleaved; into a caller's buffer too."""
    from deepseekternarized_amd import entropy

    for name, c in _cases().items():
        sym, block = c["sym"], int(c["block"][0])
        parts = {"stream": torch.from_numpy(c["stream"]).cuda(), "offsets": torch.from_numpy(c["offsets"]).cuda(), "lens": torch.from_numpy(c["lens"])}
        if "raw" in c:
            parts["raw"] = torch.from_numpy(c["raw"]).cuda()
        got = entropy.decode(parts, int(sym.size), 12, block)
        want = H.join_bytes(sym, c.get("raw"))
        assert np.array_equal(got.cpu().numpy(), want), name
        scratch = torch.full((want.size + 100,), 0xEE, dtype=torch.uint8, device="cuda")
        got2 = entropy.decode(parts, int(sym.size), 12, block, out=scratch)
        assert np.array_equal(got2.cpu().numpy(), want) and (scratch[want.size:] == 0xEE).all(), name


@pytest.mark.gpu
@pytest.mark.parametrize("n,block,two_byte", [(1, 4096, False), (4096, 4096, True), (4097, 4096, False), (1 << 20, 4096, True), (70001, 333, False), (123457, 1000, True)])
def test_device_decode_sizes_and_alignments(n, block, two_byte):
    """Round trips at block-boundary sizes, odd block lengths (unaligned stores) and a megabyte of symbols: the oracle's
    encoder (= the reference's, bit for bit) -> device decode -> the original bytes; an output view at an odd address too."""
    from deepseekternarized_amd import entropy

    rng = np.random.default_rng(n)
    if two_byte:
        w = torch.from_numpy((rng.standard_normal(n) * 0.05).astype(np.float32)).to(torch.bfloat16)
        sym, raw = H.split_bytes(w.view(torch.int16).numpy())
    else:
        sym, raw = rng.choice(64, size=n, p=np.random.default_rng(1).dirichlet(np.ones(64) * 0.2)).astype(np.uint8), None
    lens = H.code_lengths(np.bincount(sym, minlength=256))
    stream, offsets = H.huff_encode(sym, H.canonical_codes(lens), lens, block)
    parts = {"stream": torch.from_numpy(stream).cuda(), "offsets": torch.from_numpy(offsets).cuda(), "lens": torch.from_numpy(lens)}
    if raw is not None:
        parts["raw"] = torch.from_numpy(raw).cuda()
    want = H.join_bytes(sym, raw)
    got = entropy.decode(parts, n, 12, block)
    assert np.array_equal(got.cpu().numpy(), want)
    odd = torch.zeros(want.size + 3, dtype=torch.uint8, device="cuda")[3:]
    assert np.array_equal(entropy.decode(parts, n, 12, block, out=odd).cpu().numpy(), want)
    # the minimum padding the reference accepts (3 bytes past the last code's byte)
    total_bytes = (int(offsets[-1]) + 7) // 8
    parts["stream"] = torch.from_numpy(stream[: total_bytes + 3].copy()).cuda()
    if n <= (total_bytes) * 8:
        assert np.array_equal(entropy.decode(parts, n, 12, block).cpu().numpy(), want)


@pytest.mark.gpu
def test_device_decode_rejects_malformed_streams():
    """What boilerplate/kernels/csrc/huffman_validation.h and the kernel's own checks refuse: offsets outside the stream,
    blocks too short or too long for their symbol count, a truncated stream, flipped bits that desynchronise a block, a
    table entry of length 0. Nothing faults; RuntimeError every time."""
    from deepseekternarized_amd import entropy

    c = _cases()["bf16"]
    sym, block = c["sym"], int(c["block"][0])
    base = {"stream": torch.from_numpy(c["stream"]).cuda(), "offsets": torch.from_numpy(c["offsets"]).cuda(), "lens": torch.from_numpy(c["lens"]),
            "raw": torch.from_numpy(c["raw"]).cuda()}
    n = int(sym.size)

    def bad(**kw):
        p = dict(base)
        p.update(kw)
        with pytest.raises(RuntimeError):
            entropy.decode(p, n, 12, block)

    off = c["offsets"].copy(); off[2] += 1
    bad(offsets=torch.from_numpy(off).cuda())                      # block 1 ends a bit late, block 2 starts inside a code
    off = c["offsets"].copy(); off[-1] = 8 * c["stream"].size + 64
    bad(offsets=torch.from_numpy(off).cuda())                      # outside the stream
    off = c["offsets"].copy(); off[1] = off[0] + 10
    bad(offsets=torch.from_numpy(off).cuda())                      # fewer bits than symbols
    bad(stream=torch.from_numpy(c["stream"][: c["stream"].size // 2].copy()).cuda())  # truncated
    lens = c["lens"].copy()
    used = np.flatnonzero(lens)
    lens[used[np.argmax(lens[used])]] = 0                          # a used symbol loses its code: its prefix has no entry
    try:
        entropy.decode({**base, "lens": torch.from_numpy(lens)}, n, 12, block)
        raise AssertionError("expected an error")
    except (RuntimeError, ValueError):
        pass
    with pytest.raises(RuntimeError):                              # offsets of the wrong length
        entropy.decode({**base, "offsets": base["offsets"][:-1]}, n, 12, block)
    # and the good stream still decodes afterwards
    assert np.array_equal(entropy.decode(base, n, 12, block).cpu().numpy(), H.join_bytes(sym, c["raw"]))

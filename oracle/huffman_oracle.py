"""CPU oracle for Mode B's entropy decoder (canonical Huffman over weight bytes). TEST INFRASTRUCTURE ONLY.

Restates boilerplate/format/entropy.py (code lengths, canonical codes, decode table, byte split / join) and the stream
coder of boilerplate/kernels/csrc/boilerplate_cpu.cpp:130-200 (``huff_encode`` / ``huff_decode``) in NumPy / plain
Python. Only ``tests/`` imports it, as the checker of ``bp_huff_decode``; the product package never does.

Pins (tests/test_huffman.py): the reference's compiled encoder and decoder (oracle/_ref, the same file) on the same
symbols, live where that build exists and through tests/golden/huffman_ref.npz everywhere; a hand-worked stream; the
prefix property and Kraft sums of the code lengths; code lengths written by the reference's own ``code_lengths``
(in the fixture), which fixes the heap's tie-breaking.
"""

from __future__ import annotations

import heapq

import numpy as np

MAXLEN = 12
BLOCK = 4096


def code_lengths(freq, maxlen: int = MAXLEN) -> np.ndarray:
    """boilerplate/format/entropy.py:41-79: Huffman code lengths for 256 counts, limited to maxlen bits."""
    f = [int(v) for v in np.asarray(freq).tolist()]
    if len(f) != 256 or any(v < 0 for v in f):
        raise ValueError("expected 256 nonnegative integer symbol counts")
    syms = [s for s in range(256) if f[s] > 0]
    lens = [0] * 256
    if len(syms) == 1:
        lens[syms[0]] = 1
        return np.array(lens, np.uint8)
    heap = [(f[s], i, [s]) for i, s in enumerate(syms)]
    heapq.heapify(heap)
    uid = len(heap)
    while len(heap) > 1:
        a, _, sa = heapq.heappop(heap)
        b, _, sb = heapq.heappop(heap)
        for s in sa + sb:
            lens[s] += 1
        heapq.heappush(heap, (a + b, uid, sa + sb))
        uid += 1
    if syms and max(lens) > maxlen:
        for s in syms:
            lens[s] = min(lens[s], maxlen)
        kraft = sum(2.0 ** -lens[s] for s in syms)
        by_freq = sorted(syms, key=lambda s: -f[s])
        while kraft > 1.0 + 1e-12:
            for s in reversed(by_freq):
                if lens[s] < maxlen:
                    kraft -= 2.0 ** -(lens[s] + 1)
                    lens[s] += 1
                    break
    return np.array(lens, np.uint8)


def canonical_codes(lens) -> np.ndarray:
    """entropy.py:82-96: codes in order of (length, symbol), each the previous plus one, shifted to its length."""
    L = [int(v) for v in np.asarray(lens).tolist()]
    if len(L) != 256 or max(L) > MAXLEN:
        raise ValueError("expected 256 uint8 code lengths in 0..12")
    codes = [0] * 256
    code, prev = 0, 0
    for s in sorted((s for s in range(256) if L[s] > 0), key=lambda s: (L[s], s)):
        code <<= L[s] - prev
        if code >= 1 << L[s]:
            raise ValueError("oversubscribed Huffman code lengths")
        codes[s] = code
        code += 1
        prev = L[s]
    return np.array(codes, np.int32)


def decode_table(lens, maxlen: int = MAXLEN) -> np.ndarray:
    """entropy.py:99-110: [2^maxlen] int32, (symbol << 8) | length for every maxlen-bit prefix; 0 where no code starts."""
    codes = canonical_codes(lens).tolist()
    L = [int(v) for v in np.asarray(lens).tolist()]
    if max(L) > maxlen:
        raise ValueError("Huffman code length exceeds maxlen")
    lut = np.zeros(1 << maxlen, np.int32)
    for s in range(256):
        if L[s]:
            lo = codes[s] << (maxlen - L[s])
            lut[lo: lo + (1 << (maxlen - L[s]))] = (s << 8) | L[s]
    return lut


def huff_encode(sym, codes, lens, block: int = BLOCK) -> tuple[np.ndarray, np.ndarray]:
    """boilerplate_cpu.cpp:133-167: codes MSB-first back to back; offsets[b] = bit where block b starts (last = total);
    the stream is ceil(bits / 8) + 8 bytes, zero-padded."""
    sym = np.asarray(sym, np.uint8)
    L = np.asarray(lens, np.int64)[sym]
    if (L == 0).any():
        raise ValueError("Huffman symbol has no code")
    C = np.asarray(codes, np.int64)[sym]
    starts = np.concatenate([[0], np.cumsum(L)]).astype(np.int64)
    nb = -(-sym.size // block)
    offsets = np.concatenate([starts[:-1][::block][:nb], [starts[-1]]]).astype(np.int64)
    total = int(starts[-1])
    bits = np.zeros(total, np.uint8)
    for b in range(MAXLEN):  # bit b (from the code's most significant end) of every code that has one
        has = L > b
        bits[starts[:-1][has] + b] = (C[has] >> (L[has] - 1 - b)) & 1
    out = np.zeros((total + 7) // 8 + 8, np.uint8)
    packed = np.packbits(bits)  # MSB-first within a byte
    out[: packed.size] = packed
    return out, offsets


def huff_decode(stream, offsets, n: int, block: int, lut, maxlen: int = MAXLEN) -> np.ndarray:
    """boilerplate_cpu.cpp:170-200, block by block; ValueError where the reference raises."""
    stream = np.asarray(stream, np.uint8)
    off = [int(v) for v in np.asarray(offsets).tolist()]
    T = np.asarray(lut, np.int64)
    nb = -(-n // block)
    if len(off) != nb + 1 or T.size != 1 << maxlen or stream.size < 4:
        raise ValueError("incomplete Huffman metadata")
    out = np.zeros(n, np.uint8)
    data = stream.tolist()
    for b in range(nb):
        pos = off[b]
        for i in range(b * block, min(n, (b + 1) * block)):
            byte = pos >> 3
            if pos >= off[b + 1] or byte > len(data) - 4:
                raise ValueError("invalid or truncated Huffman bitstream")
            w = (data[byte] << 24) | (data[byte + 1] << 16) | (data[byte + 2] << 8) | data[byte + 3]
            peek = ((w << (pos & 7)) & 0xFFFFFFFF) >> (32 - maxlen)
            e = int(T[peek])
            length = e & 0xFF
            if not length or length > off[b + 1] - pos:
                raise ValueError("invalid or truncated Huffman bitstream")
            out[i] = e >> 8
            pos += length
        if pos != off[b + 1]:
            raise ValueError("invalid or truncated Huffman bitstream")
    return out


def split_bytes(t: np.ndarray) -> tuple[np.ndarray, np.ndarray | None]:
    """entropy.py:121-131: 1-byte elements: every byte is a symbol; 2-byte: the high byte is coded, the low one stays raw."""
    b = np.ascontiguousarray(t).view(np.uint8).reshape(-1)
    if t.dtype.itemsize == 1:
        return b, None
    if t.dtype.itemsize == 2:
        b2 = b.reshape(-1, 2)
        return np.ascontiguousarray(b2[:, 1]), np.ascontiguousarray(b2[:, 0])
    raise ValueError("Mode B codes 1- and 2-byte formats only")


def join_bytes(sym: np.ndarray, raw: np.ndarray | None) -> np.ndarray:
    """entropy.py:134-137."""
    return sym if raw is None else np.stack([raw, sym], -1).reshape(-1)

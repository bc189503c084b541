"""Writes tests/golden/huffman_ref.npz: symbols, the code lengths the REFERENCE's own `code_lengths` gives them
(boilerplate/format/entropy.py:41-79, pure Python: fixes the heap's tie-breaking), and the stream / offsets its compiled
encoder writes (boilerplate/kernels/csrc/boilerplate_cpu.cpp:133-167, through oracle/_ref), for a 1-byte and a 2-byte
format and a case where the 12-bit limit lengthens codes. Run in the build container only, after `make -C oracle ref`:

    python tests/golden/make_huffman_fixture.py [/root/reference]
"""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent))


def main() -> int:
    ref_root = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    sys.path.insert(0, str(ref_root))
    from boilerplate.format.entropy import canonical_codes, code_lengths, decode_table  # pure Python

    from _util import reference_build

    ext = reference_build()
    assert ext is not None, "build oracle/_ref first"
    rng = np.random.default_rng(0)
    cases = {}
    # bf16 weights: the coded high bytes, with the raw low bytes; blocks of 1024 so that several exist
    w = torch.from_numpy((rng.standard_normal(5000) * 0.02).astype(np.float32)).to(torch.bfloat16)
    b2 = w.view(torch.int16).numpy().view(np.uint8).reshape(-1, 2)
    cases["bf16"] = (np.ascontiguousarray(b2[:, 1]), np.ascontiguousarray(b2[:, 0]), 1024)
    # fp8-like bytes: every byte a symbol, geometric frequencies so that the 12-bit limit binds
    p = 0.5 ** np.arange(1, 41, dtype=np.float64)
    sym = rng.choice(40, size=6000, p=p / p.sum()).astype(np.uint8)
    cases["skewed"] = (sym, None, 4096)
    cases["one_symbol"] = (np.full(300, 7, np.uint8), None, 128)
    out = {}
    for name, (sym, raw, block) in cases.items():
        lens = code_lengths(torch.bincount(torch.from_numpy(sym).long(), minlength=256), 12)
        codes = canonical_codes(lens)
        stream, offsets = ext.huff_encode(torch.from_numpy(sym), codes, lens, block)
        back = ext.huff_decode(stream, offsets, sym.size, block, decode_table(lens, 12), 12)
        assert np.array_equal(back.numpy(), sym)
        out[name + ".sym"], out[name + ".lens"], out[name + ".codes"] = sym, lens.numpy(), codes.numpy()
        out[name + ".stream"], out[name + ".offsets"], out[name + ".block"] = stream.numpy(), offsets.numpy(), np.array([block])
        if raw is not None:
            out[name + ".raw"] = raw
    np.savez_compressed(HERE / "huffman_ref.npz", **out)
    print("wrote", HERE / "huffman_ref.npz")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

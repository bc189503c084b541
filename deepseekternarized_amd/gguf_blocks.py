"""Single-term ternary weights as llama.cpp ``TQ1_0`` / ``TQ2_0`` blocks, and back, on the device.

The reference converts a Mode C / D weight with k = 1, ``group: 256`` and fp16 scales by dequantizing it and calling
``gguf.quants.quantize`` (``boilerplate/format/gguf_export.py:45-58``, ``:103-114``), then verifies that the blocks
dequantize to the same values bit for bit. ``to_gguf_blocks`` makes the same blocks straight from the packed rows;
``from_gguf_blocks`` reads such blocks into a :class:`PackedTerm` of either packing. Tensor naming, the Llama Q/K row
permutation and the GGUF container (``ternary_gguf_tensors``, ``merge_into_base``) need llama.cpp's ``gguf`` package
and are not part of this path.
"""

from __future__ import annotations

import torch

from .kernels import _lib
from .kernels.ternary_hip import _fmt_code, _need_ext
from .ternary.ops import PackedTerm
from .ternary.pack import pack, packed_cols

QK = 256
_QTYPE = {"tq1": _lib.BP_GGUF_TQ1_0, "tq2": _lib.BP_GGUF_TQ2_0, "tq1_0": _lib.BP_GGUF_TQ1_0, "tq2_0": _lib.BP_GGUF_TQ2_0}


def _check(K: int, group: int, scale: torch.Tensor | None) -> None:
    """The conditions of ``_single_term`` (boilerplate/format/gguf_export.py:45-58), with its messages."""
    if group != QK or (scale is not None and scale.dtype != torch.float16):
        raise ValueError(f"group {group} / {scale.dtype if scale is not None else 'fp16'} scales (TQ needs group 256, fp16)")
    if K % QK:
        raise ValueError(f"input dim {K} not a multiple of 256")


def to_gguf_blocks(term: PackedTerm, K: int, fmt: str, group: int = QK, qtype: str = "tq1") -> torch.Tensor:
    """uint8 ``[N, K / 256 * block bytes]``: the weight's rows as TQ1_0 (54-byte) or TQ2_0 (66-byte) blocks."""
    _check(K, group, term.scale)
    e = _need_ext(term.packed)
    N = term.packed.size(0)
    if tuple(term.packed.shape) != (N, packed_cols(fmt, K)) or tuple(term.scale.shape) != (N, K // QK):
        raise ValueError("packed / scale shapes do not match K and the packing")
    q = _QTYPE[qtype]
    bs = int(e.lib.bp_gguf_block_bytes(q))
    out = torch.empty(N, K // QK * bs, dtype=torch.uint8, device=term.packed.device)
    packed, scale = term.packed.contiguous(), term.scale.contiguous()
    with torch.cuda.device(out.device):
        for r0 in range(0, N, 65535):
            r1 = min(N, r0 + 65535)
            _lib.check(e.lib.bp_gguf_from_ternary(out[r0:r1].data_ptr(), q, packed[r0:r1].data_ptr(), scale[r0:r1].data_ptr(), r1 - r0, K,
                                                  _fmt_code(fmt), _lib.stream_ptr(out.device)))
    return out


def from_gguf_blocks(blocks: torch.Tensor, K: int, fmt: str, qtype: str = "tq1") -> PackedTerm:
    """The blocks of one weight (uint8 ``[N, K / 256 * block bytes]``) as packed rows of ``fmt`` and fp16 scales ``[N, K / 256]``."""
    _check(K, QK, None)
    e = _need_ext(blocks)
    q = _QTYPE[qtype]
    bs = int(e.lib.bp_gguf_block_bytes(q))
    N = blocks.size(0)
    if blocks.dtype != torch.uint8 or blocks.dim() != 2 or blocks.size(1) != K // QK * bs:
        raise ValueError("blocks must be uint8 [N, K / 256 * block bytes]")
    blocks = blocks.contiguous()
    trits = torch.empty(N, K, dtype=torch.int8, device=blocks.device)
    scale = torch.empty(N, K // QK, dtype=torch.float16, device=blocks.device)
    with torch.cuda.device(blocks.device):
        for r0 in range(0, N, 65535):
            r1 = min(N, r0 + 65535)
            _lib.check(e.lib.bp_gguf_to_trits(trits[r0:r1].data_ptr(), scale[r0:r1].data_ptr(), blocks[r0:r1].data_ptr(), q, r1 - r0, K,
                                              _lib.stream_ptr(blocks.device)))
    return PackedTerm(pack(trits, fmt), scale)

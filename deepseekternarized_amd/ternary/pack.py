"""Ternary packing formats TQ2 and TQ1 on the device (mirror of ``boilerplate/ternary/pack.py``).

A ternary weight matrix ``T`` [N, K] with entries in {-1, 0, +1} is stored row-major, each trit as
the digit ``u = t + 1``:

* **TQ2**: ``byte = u0 | u1 << 2 | u2 << 4 | u3 << 6``; ``ceil(K / 4)`` bytes per row.
* **TQ1**: ``byte = u0 + 3 u1 + 9 u2 + 27 u3 + 81 u4`` (0..242); ``ceil(K / 5)`` bytes per row.

Rows are padded with digit 1 (trit 0). Scales are separate, one per row per ``group`` K entries.
The layout is the reference's, byte for byte; ``pack`` / ``unpack`` run as HIP kernels on device
tensors and raise for CPU tensors (this build has no CPU path).
"""

from __future__ import annotations

import torch

from ..kernels import _lib
from ..kernels.ternary_hip import _fmt_code, _need_ext

FORMATS = ("tq2", "tq1")


def bits_per_weight(fmt: str) -> float:
    """boilerplate/ternary/pack.py:26-27."""
    return {"tq2": 2.0, "tq1": 1.6}[fmt]


def packed_cols(fmt: str, K: int) -> int:
    """boilerplate/ternary/pack.py:30-31."""
    return -(-K // (4 if fmt == "tq2" else 5))


def pack(t: torch.Tensor, fmt: str) -> torch.Tensor:
    """int8 trits [N, K] -> uint8 [N, packed_cols] (boilerplate/ternary/pack.py:43-45,57-59,77-78)."""
    code = _fmt_code(fmt)
    e = _need_ext(t)
    if t.dim() != 2:
        raise RuntimeError("pack takes a [N, K] trit matrix")
    t8 = t.to(torch.int8).contiguous()
    N, K = t8.shape
    out = torch.empty(N, packed_cols(fmt, K), dtype=torch.uint8, device=t.device)
    with torch.cuda.device(t.device):
        _lib.check(e.lib.bp_pack_trits(out.data_ptr(), t8.data_ptr(), N, K, code, _lib.stream_ptr(t.device)))
    return out


def unpack(p: torch.Tensor, fmt: str, K: int) -> torch.Tensor:
    """uint8 [N, packed_cols] -> int8 trits [N, K] (boilerplate/ternary/pack.py:48-51,73-74,81-82);
    TQ2 code 3 decodes to +2 and TQ1 bytes >= 243 to 0, as in the reference."""
    code = _fmt_code(fmt)
    e = _need_ext(p)
    if p.dim() != 2 or p.dtype != torch.uint8 or p.size(1) != packed_cols(fmt, K):
        raise RuntimeError("unpack takes a uint8 [N, packed_cols(fmt, K)] matrix")
    p = p.contiguous()
    out = torch.empty(p.size(0), K, dtype=torch.int8, device=p.device)
    with torch.cuda.device(p.device):
        _lib.check(e.lib.bp_unpack_trits(out.data_ptr(), p.data_ptr(), p.size(0), K, code, _lib.stream_ptr(p.device)))
    return out


def pack_tq2(t: torch.Tensor) -> torch.Tensor:
    return pack(t, "tq2")


def pack_tq1(t: torch.Tensor) -> torch.Tensor:
    return pack(t, "tq1")


def unpack_tq2(p: torch.Tensor, K: int) -> torch.Tensor:
    return unpack(p, "tq2", K)


def unpack_tq1(p: torch.Tensor, K: int) -> torch.Tensor:
    return unpack(p, "tq1", K)


def tq1_lut(device=None) -> torch.Tensor:
    """[256, 5] int8 trits for each byte value, rows >= 243 decode to 0
    (boilerplate/ternary/pack.py:62-67), written by the device."""
    dev = torch.device(device if device is not None else "cuda")
    probe = torch.empty(0, device=dev)
    e = _need_ext(probe)
    out = torch.empty(256, 5, dtype=torch.int8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(e.lib.bp_tq1_lut(out.data_ptr(), _lib.stream_ptr(dev)))
    return out


class _LazyLut:
    """``_TQ1_LUT`` of the reference (boilerplate/ternary/pack.py:70, a module-level [256, 5] int8 tensor that
    ``ternary/ops.py:17`` imports and hands to the kernels). Here the table is produced by the device on first use,
    per device, because importing this package must not need a GPU: ``_TQ1_LUT.to(device)`` and ``_TQ1_LUT.tensor()``
    return it."""

    def __init__(self):
        self._by_device = {}

    def to(self, device=None) -> torch.Tensor:
        dev = torch.device(device if device is not None else "cuda")
        if dev.type == "cuda" and dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        if dev not in self._by_device:
            self._by_device[dev] = tq1_lut(dev)
        return self._by_device[dev]

    def tensor(self) -> torch.Tensor:
        return self.to(None)


_TQ1_LUT = _LazyLut()


def expand_scales(scale: torch.Tensor) -> torch.Tensor:
    """Stored fp16/bf16 scales -> float32 (``t.scale.float()``, boilerplate/ternary/ops.py:37)."""
    e = _need_ext(scale)
    s = scale.contiguous()
    out = torch.empty(s.shape, dtype=torch.float32, device=s.device)
    with torch.cuda.device(s.device):
        _lib.check(e.lib.bp_expand_scales(out.data_ptr(), s.data_ptr(), _lib.dtype_code(s.dtype), s.numel(),
                                          _lib.stream_ptr(s.device)))
    return out

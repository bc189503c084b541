"""Ternary linear layers (Mode C with k terms, Mode D with k = 1) on gfx950.

Mirror of ``boilerplate/ternary/ops.py``: ``quant_act_int8``, ``PackedTerm``, ``TernaryLinear``.
Activations into a ternary layer are quantized to int8 per token with an absmax scale (default) or
kept in floating point (``act="bf16"``); either way the product runs in the HIP kernels, all k terms
in one launch, with the scales read in their stored fp16/bf16 form.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from ..kernels import _lib
from ..kernels.ternary_hip import _fmt_code, _need_ext, dense_offsets, grouped_ternary_gemm


def quant_act_int8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-token absmax int8: x ~= q * s, q in [-127, 127] (boilerplate/ternary/ops.py:20-25)."""
    e = _need_ext(x)
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        x = x.float()
    x = x.contiguous()
    K = x.size(-1)
    M = x.numel() // K if K else 0
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    s = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(e.lib.bp_quant_act_int8(q.data_ptr(), s.data_ptr(), x.data_ptr(), _lib.dtype_code(x.dtype), M, K,
                                           _lib.stream_ptr(x.device)))
    return q, s


@dataclass
class PackedTerm:
    packed: torch.Tensor  # [N, ceil(K / per_byte)] uint8
    scale: torch.Tensor  # [N, G] fp16/bf16 as stored


class TernaryLinear:
    """``y = sum_terms kernel(x, term)`` (boilerplate/ternary/ops.py:34-86).

    ``backend``: ``"auto"``/``"cuda"``/``"hip"`` use the tuned kernels, ``"torch"`` the
    reference-order kernel; ``"cpp"`` (the reference's CPU kernel) does not exist in this build.
    """

    def __init__(self, terms: list[PackedTerm], K: int, fmt: str, group: int, act: str = "int8", backend: str = "auto"):
        _fmt_code(fmt)
        if act not in ("int8", "bf16"):
            raise ValueError(f"unknown activation mode {act!r}")
        self.terms, self.K, self.fmt, self.group, self.act = terms, K, fmt, group, act
        self.backend = backend
        self._dev = None

    def _on(self, device) -> list[tuple[torch.Tensor, torch.Tensor]]:
        """(packed [1, N, Kp], scale [1, N, G] as stored) per term on ``device``, copied once and kept
        (boilerplate/ternary/ops.py:41-45; the float32 scale copy of :37 is not needed here)."""
        if self._dev is None or self._dev[0] != device:
            self._dev = (device, [(t.packed.to(device).contiguous()[None], t.scale.to(device).contiguous()[None])
                                  for t in self.terms])
        return self._dev[1]

    @property
    def out_features(self) -> int:
        return self.terms[0].packed.size(0)

    def dequantized(self, device=None) -> torch.Tensor:
        """The dense float32 [N, K] weight ``sum_terms trits * scale`` (boilerplate/ternary/ops.py:51-58), computed on
        the device from the decoded trits and the widened scales (``bp_unpack_trits``, ``bp_expand_scales``) with the
        reference's operation order, and kept. ``device``: where the terms are not on a HIP device yet."""
        from .pack import expand_scales, unpack

        if getattr(self, "_deq", None) is None:
            dev = torch.device(device) if device is not None else self.terms[0].packed.device
            w = None
            for packed, scale in self._on(dev):
                d = unpack(packed[0], self.fmt, self.K).float() * expand_scales(scale[0]).repeat_interleave(self.group, -1)[:, : self.K]
                w = d if w is None else w + d
            self._deq = w
        return self._deq

    def __call__(self, x: torch.Tensor, out_dtype=torch.bfloat16) -> torch.Tensor:
        shape = x.shape
        x2 = x.reshape(-1, self.K)
        _need_ext(x2)
        terms = self._on(x2.device)
        if self.act == "int8":
            q, s = quant_act_int8(x2)
        else:
            q, s = (x2 if x2.dtype in (torch.bfloat16, torch.float16, torch.float32) else x2.float()).contiguous(), None
        out = grouped_ternary_gemm(q, s, dense_offsets(x2.device, x2.size(0)), [p for p, _ in terms], [sc for _, sc in terms],
                                   self.K, self.group, self.fmt, backend=self.backend, max_rows=x2.size(0))
        return out.view(*shape[:-1], -1).to(out_dtype)

"""Weight -> trits and scales on the device: the BitNet b1.58 absmean quantizer that produces Mode D weights.

Mirror of ``absmean_ternary`` (``boilerplate/ternary/fit.py:78-96``) and of ``BitLinear.packed_term``
(``boilerplate/qat/bitlinear.py:75-80``); both run as one HIP kernel (``bp_absmean_pack``). The other producers of the
reference (``fit_term``, ``fit_residual``, ``fit_gptq``) are export-time tooling and are not part of this build.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from ..kernels import _lib
from ..kernels.ternary_hip import _fmt_code, _need_ext
from .ops import PackedTerm
from .pack import packed_cols


@dataclass
class TernaryTerm:
    trits: torch.Tensor  # [N, K] int8 in {-1, 0, +1}
    scale: torch.Tensor  # [N, ceil(K / group)] fp16/bf16


def _absmean(weight: torch.Tensor, group: int, scale_dtype: torch.dtype, fmt: str, want_trits: bool):
    if weight.ndim != 2 or group <= 0 or weight.size(1) == 0:
        raise ValueError("weight must be a matrix with a nonempty input dimension and positive group")
    if scale_dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("scale_dtype must be float16 or bfloat16")
    e = _need_ext(weight)
    w = weight if weight.dtype in (torch.float32, torch.bfloat16, torch.float16) else weight.float()
    w = w.contiguous()
    N, K = w.shape
    dev = w.device
    packed = torch.empty(N, packed_cols(fmt, K), dtype=torch.uint8, device=dev)
    scale = torch.empty(N, math.ceil(K / group), dtype=scale_dtype, device=dev)
    trits = torch.empty(N, K, dtype=torch.int8, device=dev) if want_trits else None
    with torch.cuda.device(dev):
        _lib.check(e.lib.bp_absmean_pack(packed.data_ptr(), scale.data_ptr(), _lib.dtype_code(scale_dtype),
                                         trits.data_ptr() if trits is not None else None, w.data_ptr(), _lib.dtype_code(w.dtype),
                                         N, K, int(group), _fmt_code(fmt), _lib.stream_ptr(dev)))
    return packed, scale, trits


@torch.no_grad()
def absmean_ternary(weight: torch.Tensor, group: int, scale_dtype: torch.dtype = torch.float16) -> TernaryTerm:
    """trits = clamp(round(W / s), -1, 1) with s = mean |W| per row and group, rounded to the stored scale format
    before quantizing (boilerplate/ternary/fit.py:78-96)."""
    _, scale, trits = _absmean(weight, group, scale_dtype, "tq2", True)
    return TernaryTerm(trits, scale)


@torch.no_grad()
def packed_term(weight: torch.Tensor, group: int, fmt: str, scale_dtype: torch.dtype = torch.float16) -> PackedTerm:
    """The weight quantized and packed in the engine's TQ1 / TQ2 layout in one pass over it
    (``BitLinear.packed_term``, boilerplate/qat/bitlinear.py:75-80)."""
    if fmt not in ("tq1", "tq2"):
        raise ValueError("packing must be tq1 or tq2")
    packed, scale, _ = _absmean(weight, group, scale_dtype, fmt, False)
    return PackedTerm(packed, scale)

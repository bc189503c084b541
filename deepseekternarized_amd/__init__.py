"""MI355X (gfx950) implementation of Boilerplate's ternary expert-linear path.

Same Python-facing names as the reference (``boilerplate/kernels/ternary_cuda.py``,
``boilerplate/ternary/{ops,pack}.py``); all arithmetic runs in hand-written HIP kernels loaded from
``libbp_ternary_hip.so`` through its C ABI (``include/bp_ternary.h``). There is no CPU fallback: an
operator called without a HIP device or without the built library raises.
"""

from .kernels.ternary_hip import (ext, grouped_ternary_gemm, sort_by_expert, ternary_gemm,  # noqa: F401
                                  ternary_gemm_float, ternary_gemm_ref)
from .ternary.ops import PackedTerm, TernaryLinear, quant_act_int8  # noqa: F401
from .ternary.fit import TernaryTerm, absmean_ternary, packed_term  # noqa: F401
from .ternary.pack import (FORMATS, bits_per_weight, pack, packed_cols, tq1_lut, unpack)  # noqa: F401

__all__ = ["ext", "ternary_gemm", "ternary_gemm_float", "ternary_gemm_ref", "grouped_ternary_gemm",
           "sort_by_expert", "PackedTerm", "TernaryLinear", "quant_act_int8", "FORMATS", "bits_per_weight",
           "pack", "unpack", "packed_cols", "tq1_lut", "TernaryTerm", "absmean_ternary", "packed_term"]

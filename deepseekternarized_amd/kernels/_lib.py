"""ctypes binding of libbp_ternary_hip.so (declarations follow include/bp_ternary.h)."""

from __future__ import annotations

import ctypes as C
from functools import lru_cache
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent.parent / "libbp_ternary_hip.so"

BP_I8, BP_BF16, BP_F16, BP_F32 = 0, 1, 2, 3
BP_TQ1, BP_TQ2 = 1, 2
BP_ERR_OFFSETS = 2
BP_MAX_TERMS = 4
BP_GGUF_TQ1_0, BP_GGUF_TQ2_0 = 34, 35

_p, _i, _l = C.c_void_p, C.c_int, C.c_int64

SIGNATURES = {
    "bp_last_error": (C.c_char_p, []),
    "bp_version": (C.c_char_p, []),
    "bp_last_kernel": (C.c_char_p, []),
    "bp_set_kernel_policy": (_i, [_i]),
    "bp_reload_tuning": (None, []),
    "bp_ternary_grouped_gemm": (_i, [_p, _p, _i, _p, _p, _p, _p, _p, _i, _i, _l, _l, _l, _l, _l, _l, _l, _i, _l, _p, _p]),
    "bp_grouped_gemm_workspace_bytes": (C.c_size_t, [_i, _l, _l, _l, _l, _i, _l]),
    "bp_ternary_grouped_gemm_ws": (_i, [_p, _p, _i, _p, _p, _p, _p, _p, _i, _i, _l, _l, _l, _l, _l, _l, _l, _i, _l, _p, C.c_size_t, _p]),
    "bp_unpack_trits": (_i, [_p, _p, _l, _l, _i, _p]),
    "bp_pack_trits": (_i, [_p, _p, _l, _l, _i, _p]),
    "bp_expand_scales": (_i, [_p, _p, _i, _l, _p]),
    "bp_tq1_lut": (_i, [_p, _p]),
    "bp_quant_act_int8": (_i, [_p, _p, _p, _i, _l, _l, _p]),
    "bp_absmean_pack": (_i, [_p, _p, _i, _p, _p, _i, _l, _l, _l, _i, _p]),
    "bp_sort_workspace_ints": (_l, [_l, _l]),
    "bp_sort_by_expert": (_i, [_p, _p, _p, _l, _l, _p, _p, _p]),
    "bp_sort_by_expert_static": (_i, [_p, _p, _p, _l, _l, _p, _p]),
    "bp_check_max_rows": (_i, [_p, _p, _l, _l, _l, _p]),
    "bp_gather_rows": (_i, [_p, _p, _p, _l, _l, _l, _l, _p]),
    "bp_swiglu_bf16": (_i, [_p, _p, _p, _l, _l, _l, _p]),
    "bp_moe_combine_bf16": (_i, [_p, _p, _p, _p, _p, _l, _l, _l, _p]),
    "bp_swiglu_v4": (_i, [_p, _p, _p, _p, _p, _l, C.c_float, _l, _l, _l, _p]),
    "bp_moe_combine_v4": (_i, [_p, _i, _p, _p, _p, _l, _l, _l, _p]),
    "bp_route_topk": (_i, [_p, _i, _p, _p, _i, _l, _l, _l, _i, _p]),
    "bp_moe_layer_v4": (_i, [_p, _i, _p, _p, _p, C.c_float, _p, _p, _p, _p, _i, _i, _l, _l, _l, _l, _l, _l, _i, _i, _p, C.c_size_t, _p, _p]),
    "bp_gguf_block_bytes": (_l, [_i]),
    "bp_gguf_from_ternary": (_i, [_p, _i, _p, _p, _l, _l, _i, _p]),
    "bp_gguf_to_trits": (_i, [_p, _p, _p, _i, _l, _l, _p]),
    "bp_huff_decode": (_i, [_p, _l, _p, _l, _p, _p, _l, _l, _p, _p, _l, _p, _l, _p, _p]),
    "bp_moe_layer_workspace_bytes": (C.c_size_t, [_l, _l, _l, _l, _l, _i, _i]),
    "bp_moe_layer_bf16": (_i, [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _l, _l, _l, _l, _l, _l, _i, _i, _p, C.c_size_t, _p, _p]),
}


@lru_cache(1)
def load() -> C.CDLL:
    """The shared library, or RuntimeError when it has not been built (no silent fallback)."""
    if not LIB_PATH.exists():
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m deepseekternarized_amd.build`")
    lib = C.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


def check(rc: int) -> None:
    """Nonzero status -> the reference's error convention (RuntimeError; ValueError for offsets)."""
    if rc == 0:
        return
    msg = load().bp_last_error().decode() or f"bp_ternary error {rc}"
    if rc == BP_ERR_OFFSETS:
        raise ValueError(msg)
    raise RuntimeError(msg)


def dtype_code(dtype) -> int:
    import torch

    table = {torch.int8: BP_I8, torch.bfloat16: BP_BF16, torch.float16: BP_F16, torch.float32: BP_F32}
    if dtype not in table:
        raise RuntimeError(f"unexpected ternary GEMM dtype {dtype}")
    return table[dtype]


def stream_ptr(device) -> int:
    import torch

    return torch.cuda.current_stream(device).cuda_stream

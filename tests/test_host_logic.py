"""Python-layer conventions of the drop-in API, checked without a GPU (reference
boilerplate/kernels/ternary_cuda.py:46-49,71-77,94-97,104-105; tests/test_ternary_cuda.py:60-66)."""

import pytest
import torch

import deepseekternarized_amd as bp
from deepseekternarized_amd.kernels import ternary_hip
from deepseekternarized_amd.ternary import pack as bp_pack

needs_no_gpu = pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-device behaviour")


def test_public_names_match_the_reference_interface():
    for name in ("ext", "ternary_gemm_ref", "ternary_gemm", "grouped_ternary_gemm", "sort_by_expert", "_fmt_code"):
        assert hasattr(ternary_hip, name)
    for name in ("PackedTerm", "TernaryLinear", "quant_act_int8", "pack", "unpack", "tq1_lut", "packed_cols",
                 "bits_per_weight", "FORMATS"):
        assert hasattr(bp, name)
    for name in ("pack_tq1", "pack_tq2", "unpack_tq1", "unpack_tq2"):
        assert hasattr(bp_pack, name)


def test_format_helpers():
    assert bp.FORMATS == ("tq2", "tq1")
    assert bp.bits_per_weight("tq1") == 1.6 and bp.bits_per_weight("tq2") == 2.0
    assert [bp.packed_cols("tq2", k) for k in (1, 4, 5, 4096)] == [1, 1, 2, 1024]
    assert [bp.packed_cols("tq1", k) for k in (1, 5, 6, 7168, 2048)] == [1, 1, 2, 1434, 410]
    assert ternary_hip._fmt_code("tq1") == 1 and ternary_hip._fmt_code("tq2") == 2
    with pytest.raises(ValueError, match="unknown ternary packing"):
        ternary_hip._fmt_code("tq3")


def test_error_conventions_precede_the_device_check():
    x = torch.zeros(2, 64, dtype=torch.int8)
    xs = torch.ones(2)
    packed = torch.zeros(4, 16, dtype=torch.uint8)
    scale = torch.ones(4, 1)
    with pytest.raises(ValueError, match="unknown ternary packing"):
        bp.ternary_gemm(x, xs, packed, scale, 64, 64, "tq9")
    with pytest.raises(TypeError, match="int8"):
        bp.ternary_gemm(x.float(), xs, packed, scale, 64, 64, "tq2")
    with pytest.raises(ValueError, match="offsets"):
        bp.grouped_ternary_gemm(x, xs, [0, 1], packed[None], scale[None], 64, 64, "tq2")
    with pytest.raises(ValueError, match="offsets"):
        bp.grouped_ternary_gemm(x, xs, [0, 3, 2], torch.stack([packed, packed]), torch.stack([scale, scale]), 64, 64, "tq2")
    with pytest.raises(ValueError, match="unknown activation mode"):
        bp.TernaryLinear([bp.PackedTerm(packed, scale.half())], 64, "tq2", 64, act="fp8")


@needs_no_gpu
def test_backend_absence_is_clean():
    assert ternary_hip.ext() is None
    x = torch.zeros(2, 64, dtype=torch.int8)
    xs = torch.ones(2)
    packed = torch.zeros(4, 16, dtype=torch.uint8)
    scale = torch.ones(4, 1)
    for backend in ("cuda", "auto", "torch", "cpp"):
        with pytest.raises(RuntimeError, match="unavailable"):
            bp.ternary_gemm(x, xs, packed, scale, 64, 64, "tq2", backend=backend)
    lin = bp.TernaryLinear([bp.PackedTerm(packed, scale.half())], 64, "tq2", 64)
    assert lin.out_features == 4
    with pytest.raises(RuntimeError, match="unavailable"):  # no silent CPU fallback anywhere
        lin(torch.zeros(2, 64))
    with pytest.raises(RuntimeError, match="unavailable"):
        bp.pack(torch.zeros(2, 8, dtype=torch.int8), "tq2")
    with pytest.raises(RuntimeError, match="unavailable"):
        bp.quant_act_int8(torch.zeros(2, 8))
    with pytest.raises(RuntimeError, match="unavailable"):
        bp.sort_by_expert(torch.zeros(4, dtype=torch.int64), 2)

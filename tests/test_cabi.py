"""The C-ABI library loads without a GPU, exports every symbol include/bp_ternary.h declares, and its
argument validation (which runs before any HIP call) rejects malformed calls the way the reference's
native boundary does (reference tests/test_kernel_security.py:19-38; ternary_cuda_kernel.cu:109-141)."""

import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "bp_ternary.h"


@pytest.fixture(scope="module")
def lib():
    from deepseekternarized_amd.kernels import _lib

    if not _lib.LIB_PATH.exists():  # built only when nothing is there
        from deepseekternarized_amd.build import build

        build(verbose=False)
    return _lib.load()


def _declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(bp_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from deepseekternarized_amd.kernels import _lib

    names = _declared()
    assert "bp_ternary_grouped_gemm" in names and len(names) >= 12
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/bp_ternary.h but not exported"
    assert sorted(_lib.SIGNATURES) == names
    assert lib.bp_version().decode().endswith("gfx950")


def _gemm(lib, **over):
    """A well-formed (but pointer-fake) call; validation must fail before any pointer is used."""
    a = dict(out=8, x=8, x_dtype=0, x_scale=8, offsets=8, offsets_host=None, packed=None, w_scale=None, scale_dtype=3,
             n_terms=1, T=1, N=2, K=5, Kp=2, G=2, group=3, E=1, fmt=2, max_rows=1, lut1=None, stream=None)
    a.update(over)
    pk = (C.c_void_p * 4)(8, 8, 8, 8)
    sc = (C.c_void_p * 4)(8, 8, 8, 8)
    if a["packed"] is None:
        a["packed"] = C.cast(pk, C.c_void_p)
    if a["w_scale"] is None:
        a["w_scale"] = C.cast(sc, C.c_void_p)
    return lib.bp_ternary_grouped_gemm(*a.values())


@pytest.mark.parametrize("over", [
    dict(K=0), dict(K=2 ** 62), dict(group=0), dict(group=2 ** 25), dict(fmt=0), dict(fmt=3),
    dict(Kp=1), dict(Kp=4), dict(G=1), dict(G=3), dict(x_dtype=7), dict(scale_dtype=0), dict(scale_dtype=9),
    dict(n_terms=0), dict(n_terms=5), dict(T=-1), dict(N=-1), dict(E=70000), dict(max_rows=-1),
    dict(offsets=None), dict(out=None), dict(x=None), dict(x_scale=None), dict(packed=0), dict(w_scale=0),
])
def test_grouped_gemm_rejects_malformed_arguments(lib, over):
    rc = _gemm(lib, **over)
    assert rc == 1, over
    assert lib.bp_last_error()  # a message is available


def test_grouped_gemm_validates_host_offsets(lib):
    def call(offs, T=4, E=2, max_rows=4):
        arr = (C.c_int64 * len(offs))(*offs)
        return _gemm(lib, T=T, E=E, max_rows=max_rows, offsets_host=C.cast(arr, C.c_void_p))

    assert call([1, 2, 4]) == 2 and b"start at 0" in lib.bp_last_error()
    assert call([0, 2, 3]) == 2
    assert call([0, 3, 2, ][:3], T=2) == 2 and b"nondecreasing" in lib.bp_last_error()
    assert call([0, 1, 4], max_rows=2) == 1 and b"max_rows" in lib.bp_last_error()


def test_empty_problems_return_ok_without_a_device(lib):
    assert _gemm(lib, T=0, max_rows=0) == 0
    assert _gemm(lib, N=0) == 0
    assert _gemm(lib, E=0, offsets=None) == 0


def test_other_entry_points_validate(lib):
    assert lib.bp_unpack_trits(8, 8, 1, 0, 2, None) == 1
    assert lib.bp_unpack_trits(8, 8, 1, 5, 3, None) == 1
    assert lib.bp_unpack_trits(None, 8, 1, 5, 2, None) == 1
    assert lib.bp_pack_trits(8, 8, -1, 5, 2, None) == 1
    assert lib.bp_unpack_trits(8, 8, 0, 5, 2, None) == 0  # nothing to do
    assert lib.bp_expand_scales(8, 8, 0, 4, None) == 1  # int8 is not a scale dtype
    assert lib.bp_quant_act_int8(8, 8, 8, 0, 1, 4, None) == 1  # int8 input is not quantisable
    assert lib.bp_quant_act_int8(8, 8, 8, 3, 1, 0, None) == 1
    assert lib.bp_gather_rows(8, 8, 8, 0, 1, 1, 4, None) == 1  # divisor 0
    assert lib.bp_gather_rows(8, 8, 8, 1, 1, 1, 3, None) == 1  # odd row size
    assert lib.bp_sort_by_expert(8, 8, 8, -1, 4, None, None, None) == 1
    assert lib.bp_sort_by_expert(8, 8, 8, 4, 1 << 20, None, None, None) == 1  # needs a workspace
    assert lib.bp_sort_workspace_ints(100, 64) == 0 and lib.bp_sort_workspace_ints(100, 4096) == 16 * 4096
    assert lib.bp_swiglu_bf16(8, 8, 8, 1, 4, 2, None) == 1
    assert lib.bp_moe_combine_bf16(8, 8, 8, 8, 8, 1, 65, 4, None) == 1
    assert lib.bp_set_kernel_policy(1) == 0 and lib.bp_set_kernel_policy(0) == 1

"""Checks both oracle restatements against the reference's OWN CPU kernel: through the committed
fixture written from it (tests/golden/ref_cpu_kernel.npz) and, where oracle/_ref is loadable, live.

Tolerances are the reference's own between its backends: rtol 1e-5 / atol 1e-4 for the int8 path
(reference tests/test_ternary_cuda.py:34-37), rtol 1e-4 / atol 1e-3 for float activations
(tests/test_ternary.py:98)."""

import numpy as np
import pytest

from _util import c_gemm, golden, oracle_c, orc, ref_gemm, reference_build


def _terms(c):
    return [(c[f"packed{t}"], c[f"scale{t}"].astype(np.float32)) for t in range(c["terms"])]


@pytest.mark.parametrize("name", sorted(golden()))
def test_numpy_oracle_matches_reference_fixture(name):
    c = golden()[name]
    if c["int8"]:
        got = sum(orc.ternary_gemm_ref(c["x"], c["x_scale"], p, s, c["K"], c["group"], c["fmt"]) for p, s in _terms(c))
        np.testing.assert_allclose(got, c["out"], rtol=1e-5, atol=1e-4)
    else:
        got = sum(orc.ternary_gemm_float_ref(c["x"], p, s, c["K"], c["group"], c["fmt"]) for p, s in _terms(c))
        np.testing.assert_allclose(got, c["out"], rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("name", sorted(golden()))
def test_c_port_matches_reference_fixture(name):
    c = golden()[name]
    out = np.zeros((c["M"], c["N"]), np.float32)
    for p, s in _terms(c):  # accumulates in place, like stacked terms on the reference CPU path
        c_gemm(c["x"], c["x_scale"], p, s, c["K"], c["group"], c["fmt"], out=out)
    tol = dict(rtol=1e-5, atol=1e-4) if c["int8"] else dict(rtol=1e-4, atol=1e-3)
    np.testing.assert_allclose(out, c["out"], **tol)


@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_c_port_unpack_is_bit_exact(fmt):
    rng = np.random.default_rng(2)
    N, K = 13, 257
    packed = rng.integers(0, 256, (N, orc.packed_cols(fmt, K)), dtype=np.uint8)  # all byte values, incl. invalid ones
    trits = np.zeros((N, K), np.int8)
    lut = np.ascontiguousarray(orc.tq1_lut())
    assert oracle_c().bp_oracle_unpack(trits.ctypes.data, packed.ctypes.data, N, K, 1 if fmt == "tq1" else 2, lut.ctypes.data) == 0
    assert np.array_equal(trits, orc.unpack(packed, fmt, K))


def test_c_port_rejects_bad_dims():
    h = oracle_c()
    z = np.zeros(8, np.float32)
    for K, group, fmt in ((0, 3, 2), (2 ** 62, 3, 2), (5, 0, 2), (5, 3, 0)):
        assert h.bp_oracle_ternary_gemm(z.ctypes.data, z.ctypes.data, 0, z.ctypes.data, z.ctypes.data, z.ctypes.data,
                                        1, 1, K, group, fmt, z.ctypes.data, 1) == 1


@pytest.mark.skipif(reference_build() is None, reason="oracle/_ref (the reference's compiled CPU kernel) is not loadable here")
@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
@pytest.mark.parametrize("act", ["int8", "f32"])
def test_live_reference_kernel_agrees(fmt, act):
    rng = np.random.default_rng(hash((fmt, act)) % 1000)
    N, K, group, M = 33, 643, 128, 7
    trits = rng.integers(-1, 2, (N, K)).astype(np.int8)
    packed = orc.pack(trits, fmt)
    scale = (rng.random((N, -(-K // group))) + 0.01).astype(np.float16).astype(np.float32)
    xf = rng.standard_normal((M, K)).astype(np.float32)
    if act == "int8":
        x, xs = orc.quant_act_int8(xf)
        want = orc.ternary_gemm_ref(x, xs, packed, scale, K, group, fmt)
        tol = dict(rtol=1e-5, atol=1e-4)
    else:
        x, xs = xf, None
        want = orc.ternary_gemm_float_ref(x, packed, scale, K, group, fmt)
        tol = dict(rtol=1e-4, atol=1e-3)
    ref = ref_gemm(x, xs, packed, scale, K, group, fmt)
    np.testing.assert_allclose(ref, want, **tol)
    np.testing.assert_allclose(c_gemm(x, xs, packed, scale, K, group, fmt), ref, **tol)

"""Shared test helpers: oracle loaders (NumPy, plain-C port, reference build) and seeded inputs.

The oracle modules are imported here, in tests only, as the checker of the HIP path.
"""

from __future__ import annotations

import ctypes as C
import importlib.util
import subprocess
import sys
from functools import lru_cache
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
ORACLE_DIR = ROOT / "oracle"
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from oracle import ternary_oracle as orc  # noqa: E402

FMT_CODE = {"tq1": 1, "tq2": 2}


@lru_cache(1)
def oracle_c():
    """The plain-C port (oracle/ternary_cpu.c). Loaded if built; compiled only when nothing is there."""
    lib = ORACLE_DIR / "libbp_oracle_cpu.so"
    if not lib.exists():
        subprocess.run(["make", "-C", str(ORACLE_DIR), "libbp_oracle_cpu.so"], check=True, capture_output=True)
    h = C.CDLL(str(lib))
    p, l, i = C.c_void_p, C.c_int64, C.c_int
    h.bp_oracle_ternary_gemm.restype = i
    h.bp_oracle_ternary_gemm.argtypes = [p, p, i, p, p, p, l, l, l, l, i, p, i]
    h.bp_oracle_unpack.restype = i
    h.bp_oracle_unpack.argtypes = [p, p, l, l, i, p]
    h.bp_oracle_max_threads.restype = i
    return h


def c_gemm(x, x_scale, packed, w_scale, K, group, fmt, out=None, threads=0):
    """oracle/ternary_cpu.c::bp_oracle_ternary_gemm on NumPy arrays; returns out [M, N] float32."""
    h = oracle_c()
    x = np.ascontiguousarray(x)
    is_i8 = x.dtype == np.int8
    if not is_i8:
        x = np.ascontiguousarray(x, dtype=np.float32)
    M, N = x.shape[0], packed.shape[0]
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    ws = np.ascontiguousarray(w_scale, dtype=np.float32)
    xs = np.ascontiguousarray(x_scale if x_scale is not None else np.ones(M), dtype=np.float32)
    lut = np.ascontiguousarray(orc.tq1_lut())
    if out is None:
        out = np.zeros((M, N), dtype=np.float32)
    rc = h.bp_oracle_ternary_gemm(out.ctypes.data, x.ctypes.data, int(is_i8), xs.ctypes.data, packed.ctypes.data,
                                  ws.ctypes.data, M, N, K, group, FMT_CODE[fmt], lut.ctypes.data, threads)
    if rc:
        raise RuntimeError(f"bp_oracle_ternary_gemm failed with {rc}")
    return out


@lru_cache(1)
def reference_build():
    """The reference's own CPU kernel compiled into oracle/_ref (or None when that build is absent,
    or cannot be loaded on this machine)."""
    so = ORACLE_DIR / "_ref" / "boilerplate_cpu_ref.so"
    if not so.exists():
        return None
    try:
        import torch  # noqa: F401  (the module links against libtorch)

        spec = importlib.util.spec_from_file_location("boilerplate_cpu_ref", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        return mod
    except Exception:  # pragma: no cover - depends on the host
        return None


def ref_gemm(x, x_scale, packed, w_scale, K, group, fmt, out=None):
    """reference boilerplate_cpu.cpp::ternary_gemm (compiled) on NumPy arrays."""
    import torch

    mod = reference_build()
    x = np.ascontiguousarray(x)
    xt = torch.from_numpy(x if x.dtype == np.int8 else x.astype(np.float32))
    M, N = x.shape[0], packed.shape[0]
    o = torch.zeros(M, N) if out is None else torch.from_numpy(out)
    xs = torch.from_numpy(np.ascontiguousarray(x_scale if x_scale is not None else np.ones(M), dtype=np.float32))
    mod.ternary_gemm(o, xt, xs, torch.from_numpy(np.ascontiguousarray(packed)),
                     torch.from_numpy(np.ascontiguousarray(w_scale, dtype=np.float32)), K, group, FMT_CODE[fmt],
                     torch.from_numpy(orc.tq1_lut()))
    return o.numpy()


# --------------------------------------------------------------------------- seeded synthetic inputs
def synth_trits(rng, shape):
    """iid trits with P(-1) = P(+1) = 0.33, P(0) = 0.34."""
    u = rng.random(shape, dtype=np.float32)
    return np.where(u < 0.33, -1, np.where(u < 0.66, 1, 0)).astype(np.int8)


def synth_weights(seed, E, N, K, group, fmt, terms=1, second_scale=0.25):
    """Draw order: for each term: trits (E, N, K) then scales (E, N, G) = fp16(0.02 * |N(0, 1)|);
    later terms' scales are `second_scale` times the first term's (stacked residual)."""
    rng = np.random.default_rng(seed)
    G = -(-K // group)
    packed, scales = [], []
    base = None
    for t in range(terms):
        tr = synth_trits(rng, (E, N, K))
        sc = (0.02 * np.abs(rng.standard_normal((E, N, G)))).astype(np.float16)
        if t == 0:
            base = sc
        else:
            sc = (base.astype(np.float32) * second_scale).astype(np.float16)
        packed.append(np.stack([orc.pack(tr[e], fmt) for e in range(E)]))
        scales.append(sc)
    return packed, scales


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d else float(np.linalg.norm(a - b))


# --------------------------------------------------------------------------- golden fixtures
@lru_cache(1)
def golden():
    """tests/golden/ref_cpu_kernel.npz: inputs and outputs of the reference's compiled CPU kernel."""
    z = np.load(ROOT / "tests" / "golden" / "ref_cpu_kernel.npz", allow_pickle=False)
    cases = {}
    for key in z.files:
        name, field = key.rsplit(".", 1)
        cases.setdefault(name, {})[field] = z[key]
    for c in cases.values():
        N, K, group, M, terms, code, is_i8 = (int(v) for v in c["meta"])
        c.update(N=N, K=K, group=group, M=M, terms=terms, fmt="tq1" if code == 1 else "tq2", int8=bool(is_i8))
    return cases

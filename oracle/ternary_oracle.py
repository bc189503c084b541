"""CPU oracle for the ternary expert-linear path. TEST INFRASTRUCTURE ONLY.

NumPy restatement of the reference's algorithm, function by function; each function cites the
reference lines it follows. Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import this module, and only as the checker: the product package
(``deepseekternarized_amd``) never imports it and has no CPU fallback.

How each function is pinned (``tests/test_oracle.py``, ``tests/test_oracle_vs_reference_build.py``):

* pack/unpack/LUT: literal byte vectors written out by hand from the format definition
  (``boilerplate/ternary/pack.py:7-16``, ``docs/architecture/format.md:94-104``), the exhaustive
  243-pattern enumeration (``tests/test_ternary.py:23-29``), round trips at the reference's K list
  (``tests/test_ternary.py:14-20``), and a pure-Python digit-by-digit brute force.
* quant_act_int8: the reference's invariant (``tests/test_ternary.py:78-82``) plus hand-computed rows.
* ternary_gemm_ref: exact-integer special case (scale = 1, one group -> integer matmul), the dense
  fp64 product (``tests/test_ternary_cuda.py:21-36``), and the reference's compiled CPU kernel
  (``oracle/_ref``) on the reference's own test shapes.
* sort_by_expert / grouped: counting-sort definition and per-expert equivalence
  (``tests/test_ternary_cuda.py:41-57``).
* moe_layer_ref: per-token dense recomputation in float64 (no library MoE to compare against; the
  rounding points follow ``boilerplate/engine/standard.py:151-176``).

* moe_layer_v4_ref / moe_layer_ref: the reference's lines restated with torch CPU ops (bf16 tensors, softmax, topk,
  F.silu, index_add_) on dequantized weights: agreement within one bf16 step per element, nearly all equal
  (``tests/test_oracle.py``); ``topk_desc`` against ``torch.topk``.
* absmean_ternary: the reference's known-answer test, the reference's own Mode D export (``tests/golden/export_tiny``)
  bit for bit, and the literal formula in torch with the measured rate at which summation order moves a scale.

PARITY UNPINNED: ``gguf_quantize`` / ``gguf_dequantize`` (ggml TQ1_0 / TQ2_0 blocks). The reference calls the ``gguf``
package for them, which is neither vendored in the reference nor installed here; they restate llama.cpp's published
block layout and are pinned only by hand-worked blocks and the exact round trip the reference's test asks for.
Every other function here is pinned as listed.
"""

from __future__ import annotations

import numpy as np

FORMATS = ("tq2", "tq1")
_POW3 = np.array([1, 3, 9, 27, 81], dtype=np.int32)


# --------------------------------------------------------------------------- format helpers
def bits_per_weight(fmt: str) -> float:
    """boilerplate/ternary/pack.py:26-27."""
    return {"tq2": 2.0, "tq1": 1.6}[fmt]


def trits_per_byte(fmt: str) -> int:
    return 4 if fmt == "tq2" else 5


def packed_cols(fmt: str, K: int) -> int:
    """boilerplate/ternary/pack.py:30-31: bytes per packed row."""
    return -(-K // trits_per_byte(fmt))


def _digits(t: np.ndarray, per: int) -> np.ndarray:
    """boilerplate/ternary/pack.py:34-40: digits u = t + 1, row padded with digit 1 (trit 0)."""
    t = np.asarray(t)
    N, K = t.shape
    pad = -K % per
    u = (t.astype(np.int16) + 1).astype(np.uint8)
    if pad:
        u = np.concatenate([u, np.ones((N, pad), dtype=np.uint8)], axis=1)
    return u.reshape(N, -1, per)


def pack_tq2(t: np.ndarray) -> np.ndarray:
    """boilerplate/ternary/pack.py:43-45: byte = u0 | u1<<2 | u2<<4 | u3<<6."""
    u = _digits(t, 4).astype(np.int32)
    return (u[..., 0] | (u[..., 1] << 2) | (u[..., 2] << 4) | (u[..., 3] << 6)).astype(np.uint8)


def unpack_tq2(p: np.ndarray, K: int) -> np.ndarray:
    """boilerplate/ternary/pack.py:48-51: ((b >> s) & 3) - 1; code 3 decodes to +2."""
    b = np.asarray(p).astype(np.int16)
    u = np.stack([(b >> s) & 3 for s in (0, 2, 4, 6)], axis=-1).reshape(b.shape[0], -1)
    return (u[:, :K] - 1).astype(np.int8)


def pack_tq1(t: np.ndarray) -> np.ndarray:
    """boilerplate/ternary/pack.py:57-59: byte = sum_i u_i * 3**i (0..242)."""
    u = _digits(t, 5).astype(np.int32)
    return (u * _POW3).sum(-1).astype(np.uint8)


def tq1_lut() -> np.ndarray:
    """boilerplate/ternary/pack.py:62-67: [256, 5] int8, rows >= 243 decode to 0."""
    v = np.arange(256, dtype=np.int32)
    d = np.stack([(v // int(p)) % 3 for p in _POW3], axis=-1) - 1
    d[243:] = 0
    return d.astype(np.int8)


_TQ1_LUT = tq1_lut()


def unpack_tq1(p: np.ndarray, K: int) -> np.ndarray:
    """boilerplate/ternary/pack.py:73-74."""
    p = np.asarray(p)
    return _TQ1_LUT[p.astype(np.int64)].reshape(p.shape[0], -1)[:, :K]


def pack(t: np.ndarray, fmt: str) -> np.ndarray:
    """boilerplate/ternary/pack.py:77-78."""
    return pack_tq2(t) if fmt == "tq2" else pack_tq1(t)


def unpack(p: np.ndarray, fmt: str, K: int) -> np.ndarray:
    """boilerplate/ternary/pack.py:81-82."""
    return unpack_tq2(p, K) if fmt == "tq2" else unpack_tq1(p, K)


# --------------------------------------------------------------------------- bf16 / fp16 helpers
def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even) -> float32, the rounding of ``tensor.to(bfloat16)``."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    out = r.view(np.float32).copy()
    nan = np.isnan(a)
    out[nan] = np.nan
    return out.reshape(a.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), ties to even."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# --------------------------------------------------------------------------- activations
def quant_act_int8(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """boilerplate/ternary/ops.py:20-25: per-row absmax int8, fp32 arithmetic, round half to even."""
    xf = np.asarray(x, dtype=np.float32)
    amax = np.abs(xf).max(axis=-1, keepdims=True) if xf.shape[-1] else np.zeros(xf.shape[:-1] + (1,), np.float32)
    s = np.maximum((amax / np.float32(127.0)).astype(np.float32), np.float32(1e-8))
    q = np.clip(np.rint((xf / s).astype(np.float32)), -127, 127).astype(np.int8)
    return q, s[..., 0]


# --------------------------------------------------------------------------- GEMM reference
def absmean_ternary(weight: np.ndarray, group: int, scale_dtype: str = "f16") -> tuple[np.ndarray, np.ndarray]:
    """BitNet b1.58 absmean quantizer (boilerplate/ternary/fit.py:78-96): per row and group of `group` columns (the
    last group may be shorter and counts its own columns) s = scale_dtype(sum |w| / count), then
    trits = s > 0 ? clamp(rint(w / max(s, 1e-30)), -1, 1) : 0 in float32. Returns (trits int8 [N, K], scale as float32
    holding the fp16 / bf16-rounded values [N, G]).

    The float32 sum is taken in ascending column order here; the reference's ``torch.sum`` leaves the order to the
    library, so a scale could differ in its last stored bit where the sum lands within one float32 rounding of a
    fp16 rounding boundary. Pinned by the literal known-answer test of the reference (tests/test_qat.py:11-17: short
    last group, all-zero row) and by exact small-integer cases where the order cannot matter."""
    w = np.asarray(weight, np.float32)
    if w.ndim != 2 or group <= 0 or w.shape[1] == 0:
        raise ValueError("weight must be a matrix with a nonempty input dimension and positive group")
    if scale_dtype not in ("f16", "bf16"):
        raise ValueError("scale_dtype must be float16 or bfloat16")
    N, K = w.shape
    G = -(-K // group)
    scale = np.zeros((N, G), np.float32)
    trits = np.zeros((N, K), np.int8)
    for g in range(G):
        k0, k1 = g * group, min(K, (g + 1) * group)
        a = np.abs(w[:, k0:k1])
        total = np.add.accumulate(a, axis=1, dtype=np.float32)[:, -1]  # sequential float32 sum
        mean = (total / np.float32(k1 - k0)).astype(np.float32)
        s = mean.astype(np.float16).astype(np.float32) if scale_dtype == "f16" else bf16_round(mean)
        scale[:, g] = s
        q = np.rint(w[:, k0:k1] / np.maximum(s, np.float32(1e-30))[:, None]).clip(-1, 1)
        trits[:, k0:k1] = np.where(s[:, None] > 0, q, 0).astype(np.int8)
    return trits, scale


def _fmt_check(fmt: str) -> None:
    """boilerplate/kernels/ternary_cuda.py:46-49."""
    if fmt not in ("tq1", "tq2"):
        raise ValueError(f"unknown ternary packing {fmt!r}")


def group_sums_int(x: np.ndarray, packed: np.ndarray, K: int, group: int, fmt: str) -> np.ndarray:
    """Exact integer group sums acc[m, n, g] = sum_{k in g} x[m,k] * trit[n,k] (int64)."""
    t = unpack(packed, fmt, K).astype(np.int64)
    xs = np.asarray(x).astype(np.int64)
    G = -(-K // group)
    acc = np.zeros((xs.shape[0], t.shape[0], G), dtype=np.int64)
    for g in range(G):
        k0, k1 = g * group, min(K, (g + 1) * group)
        acc[:, :, g] = xs[:, k0:k1] @ t[:, k0:k1].T
    return acc


def ternary_gemm_ref(x, x_scale, packed, w_scale, K: int, group: int, fmt: str) -> np.ndarray:
    """boilerplate/kernels/ternary_cuda.py:52-64, operation for operation.

    Integer group sums are exact; then, in float32 and in ascending group order,
    ``out += float32(acc) * w_scale[:, g]`` (multiply, then add, each rounded), and finally
    ``out * x_scale[:, None]``. NumPy float32 arithmetic does not contract to FMA, like the
    reference's separate torch ops.
    """
    _fmt_check(fmt)
    acc = group_sums_int(x, packed, K, group, fmt)
    ws = np.asarray(w_scale, dtype=np.float32)
    out = np.zeros(acc.shape[:2], dtype=np.float32)
    for g in range(ws.shape[1]):
        if g * group >= K:
            break
        out += acc[:, :, g].astype(np.float32) * ws[None, :, g]
    return out * np.asarray(x_scale, dtype=np.float32)[:, None]


def ternary_gemm_float_ref(x, packed, w_scale, K: int, group: int, fmt: str) -> np.ndarray:
    """Float-activation contract of the CPU kernel (boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77,
    :114-124): y[m,n] = sum_g s[n,g] * sum_{k in g} x[m,k] * trit[n,k], x_scale ignored.

    Evaluated in float64 (the mathematically exact value up to 1e-16), so every float32 summation
    order a backend may choose lies within float32 rounding of it. Returned as float64.
    """
    _fmt_check(fmt)
    t = unpack(packed, fmt, K).astype(np.float64)
    xs = np.asarray(x, dtype=np.float64)
    ws = np.asarray(w_scale, dtype=np.float64)
    w = t * np.repeat(ws, group, axis=1)[:, :K]
    return xs @ w.T


def dequantize(terms, K: int, group: int, fmt: str) -> np.ndarray:
    """boilerplate/ternary/ops.py:51-58: W = sum_i unpack(packed_i) * scale_i (float32)."""
    w = None
    for packed, scale in terms:
        s = np.repeat(np.asarray(scale, dtype=np.float32), group, axis=1)[:, :K]
        d = unpack(packed, fmt, K).astype(np.float32) * s
        w = d if w is None else w + d
    return w


def sort_by_expert(expert_ids: np.ndarray, n_experts: int) -> tuple[np.ndarray, np.ndarray]:
    """boilerplate/kernels/ternary_cuda.py:114-118: stable argsort + bincount + cumsum."""
    ids = np.asarray(expert_ids, dtype=np.int64)
    order = np.argsort(ids, kind="stable")
    counts = np.bincount(ids, minlength=n_experts).astype(np.int64)
    return order, np.concatenate([np.zeros(1, np.int64), np.cumsum(counts)])


def check_offsets(offsets, E: int, T: int) -> np.ndarray:
    """boilerplate/kernels/ternary_cuda.py:94-97."""
    offs = np.asarray(offsets, dtype=np.int64)
    if offs.size != E + 1 or int(offs[0]) != 0 or int(offs[-1]) != T or bool((np.diff(offs) < 0).any()):
        raise ValueError("offsets must be nondecreasing, start at 0, end at the row count, one per expert + 1")
    return offs


def grouped_ternary_gemm_ref(x, x_scale, offsets, packed, w_scale, K: int, group: int, fmt: str) -> np.ndarray:
    """boilerplate/kernels/ternary_cuda.py:90-111 (the loop over non-empty experts)."""
    _fmt_check(fmt)
    E = packed.shape[0]
    offs = check_offsets(offsets, E, x.shape[0])
    out = np.zeros((x.shape[0], packed.shape[1]), dtype=np.float32)
    for e in range(E):
        a, b = int(offs[e]), int(offs[e + 1])
        if a < b:
            out[a:b] = ternary_gemm_ref(x[a:b], x_scale[a:b], packed[e], w_scale[e], K, group, fmt)
    return out


def grouped_ternary_gemm_float_ref(x, offsets, packed_terms, scale_terms, K: int, group: int, fmt: str) -> np.ndarray:
    """Grouped float-activation product with stacked terms, float64: sum over terms of the
    per-expert float contract (boilerplate/ternary/ops.py:75-79 accumulates terms into one output)."""
    E = packed_terms[0].shape[0]
    offs = check_offsets(offsets, E, x.shape[0])
    out = np.zeros((x.shape[0], packed_terms[0].shape[1]), dtype=np.float64)
    for e in range(E):
        a, b = int(offs[e]), int(offs[e + 1])
        if a < b:
            for p, s in zip(packed_terms, scale_terms):
                out[a:b] += ternary_gemm_float_ref(x[a:b], p[e], s[e], K, group, fmt)
    return out


def ternary_linear_ref(x, terms, K: int, group: int, fmt: str, act: str = "int8") -> np.ndarray:
    """boilerplate/ternary/ops.py:60-86 up to (not including) the final cast: float64 value of
    sum over terms of kernel(x, term). ``terms`` = [(packed [N,Kp] u8, scale [N,G] fp16-valued)]."""
    x2 = np.asarray(x, dtype=np.float32).reshape(-1, K)
    out = np.zeros((x2.shape[0], terms[0][0].shape[0]), dtype=np.float64)
    if act == "int8":
        q, s = quant_act_int8(x2)
        for packed, scale in terms:
            out += ternary_gemm_ref(q, s, packed, np.asarray(scale, np.float32), K, group, fmt).astype(np.float64)
    else:
        for packed, scale in terms:
            out += ternary_gemm_float_ref(x2, packed, np.asarray(scale, np.float32), K, group, fmt)
    return out


# --------------------------------------------------------------------------- MoE layer
def softmax_f32(z: np.ndarray) -> np.ndarray:
    z = np.asarray(z, dtype=np.float32)
    m = z.max(axis=-1, keepdims=True)
    e = np.exp((z - m).astype(np.float32)).astype(np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def topk_desc(scores: np.ndarray, k: int) -> tuple[np.ndarray, np.ndarray]:
    """Largest k per row, descending, ties to the lower index (a stable sort of -scores)."""
    idx = np.argsort(-scores, axis=-1, kind="stable")[:, :k]
    return np.take_along_axis(scores, idx, axis=-1), idx


def silu(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float64)
    return x / (1.0 + np.exp(-x))


def moe_layer_ref(x_bf16, router_logits, experts, top_k: int, K_hidden: int, K_inter: int, group: int, fmt: str,
                  act: str = "bf16", renorm: bool = False) -> np.ndarray:
    """boilerplate/engine/standard.py:151-176 with bf16 activations.

    ``experts[e] = (gate_terms, up_terms, down_terms)``; each ``*_terms`` a list of (packed, scale).
    Rounding points as in the reference: softmax in float32, routing weights cast to bf16, every
    linear returns bf16 (``_Linear.__call__`` passes ``out_dtype=x.dtype``, standard.py:52), silu and
    the product are bf16 ops, the weighted result is bf16, and ``index_add_`` accumulates in bf16 in
    ascending expert order.
    """
    x = bf16_round(np.asarray(x_bf16, dtype=np.float32))
    scores = softmax_f32(router_logits)
    values, indices = topk_desc(scores, top_k)
    if renorm:
        values = (values / values.sum(-1, keepdims=True, dtype=np.float32)).astype(np.float32)
    values = bf16_round(values)
    out = np.zeros_like(x)
    for e in range(len(experts)):
        token, slot = np.nonzero(indices == e)
        if token.size == 0:
            continue
        gate_t, up_t, down_t = experts[e]
        xe = x[token]
        g = bf16_round(ternary_linear_ref(xe, gate_t, K_hidden, group, fmt, act).astype(np.float32))
        u = bf16_round(ternary_linear_ref(xe, up_t, K_hidden, group, fmt, act).astype(np.float32))
        h = bf16_round((bf16_round(silu(g).astype(np.float32)) * u).astype(np.float32))
        d = bf16_round(ternary_linear_ref(h, down_t, K_inter, group, fmt, act).astype(np.float32))
        r = bf16_round((d * values[token, slot, None]).astype(np.float32))
        for i, tok in enumerate(token):  # index_add_ in bf16, one (token, slot) pair at a time
            out[tok] = bf16_round(out[tok] + r[i])
    return out


def moe_layer_v4_ref(x_bf16, weights, indices, experts, K_hidden: int, K_inter: int, group: int, fmt: str,
                     act: str = "bf16", swiglu_limit: float = 0.0) -> np.ndarray:
    """boilerplate/engine/model.py:376-387 (``swiglu``) and :407-420 (``moe``, the routed experts; the shared experts
    of :421 are further ``swiglu`` calls without weights and stay with the caller). Returns the float32 ``y``.

    ``weights`` float32 [T, k] and ``indices`` int [T, k] are the router's output (:389-405).
    Rounding points: ``w1(x)`` / ``w3(x)`` return bf16 (TernaryLinear's ``out_dtype``, boilerplate/ternary/ops.py:60) and are
    widened to float32; ``up`` is clamped to [-limit, limit] and ``gate`` to at most limit when limit > 0; ``silu(gate) * up``
    and the product with the routing weight are float32; that is rounded to bf16 once (``x.to(dtype)``) as ``w2``'s input;
    ``w2`` returns bf16; ``y[idx] +=`` accumulates in float32, experts in ascending order.
    """
    x = bf16_round(np.asarray(x_bf16, dtype=np.float32))
    weights = np.asarray(weights, dtype=np.float32)
    indices = np.asarray(indices)
    y = np.zeros_like(x, dtype=np.float32)
    lim = np.float32(swiglu_limit)
    for e in range(len(experts)):
        token, slot = np.nonzero(indices == e)
        if token.size == 0:
            continue
        gate_t, up_t, down_t = experts[e]
        xe = x[token]
        g = bf16_round(ternary_linear_ref(xe, gate_t, K_hidden, group, fmt, act).astype(np.float32))
        u = bf16_round(ternary_linear_ref(xe, up_t, K_hidden, group, fmt, act).astype(np.float32))
        if lim > 0:
            u = np.clip(u, -lim, lim)
            g = np.minimum(g, lim)
        sg = (g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float32)  # float32 silu, correctly rounded
        h = (sg * u).astype(np.float32)
        h = (weights[token, slot, None] * h).astype(np.float32)
        d = bf16_round(ternary_linear_ref(bf16_round(h), down_t, K_inter, group, fmt, act).astype(np.float32))
        for i, tok in enumerate(token):
            y[tok] = (y[tok] + d[i]).astype(np.float32)
    return y


# --------------------------------------------------------------------------- ggml TQ1_0 / TQ2_0 blocks (GGUF interop)
# boilerplate/format/gguf_export.py:103-114 (`quantize_exact`) hands the dequantized values of a single-term, group-256,
# fp16-scale ternary weight to `gguf.quants.quantize(arr, TQ1_0 | TQ2_0)` of the `gguf` Python package (llama.cpp's
# gguf-py; the reference asks for `pip install gguf` without a version) and checks that `gguf.quants.dequantize` gives
# the values back bit for bit. That package is not vendored in the reference and is absent here, so the functions
# below restate the published block layout and algorithm of llama.cpp (ggml/src/ggml-common.h `block_tq1_0` /
# `block_tq2_0`, ggml/src/ggml-quants.c `quantize_row_tq{1,2}_0_ref` / `dequantize_row_tq{1,2}_0`), which gguf-py's
# quants.py mirrors. PARITY UNPINNED against the package itself: pinned by hand-worked blocks from those formulas, the
# exhaustive digit round trip and the exact value round trip the reference's own test asks for
# (tests/test_gguf_export.py:54-75), nothing more.
GGUF_QK = 256
GGUF_TQ1_0_BYTES = 54  # qs[48] (5 trits per byte) + qh[4] (4 trits per byte) + fp16 d
GGUF_TQ2_0_BYTES = 66  # qs[64] (4 trits per byte) + fp16 d


def _gguf_digits(values: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per block of 256: d = fp16(max |x|), digits xi = lroundf(x * (1 / d)) + 1 in 0..2 (d = 0: all 1)."""
    v = np.asarray(values, np.float32)
    if v.ndim != 2 or v.shape[1] % GGUF_QK:
        raise ValueError("values must be [N, K] with K a multiple of 256")
    blk = v.reshape(v.shape[0], -1, GGUF_QK)
    d = np.abs(blk).max(-1).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d > 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    t = (blk * inv[..., None]).astype(np.float32)
    xi = (np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))).astype(np.int64) + 1  # lroundf: halves away from zero
    return d.astype(np.float16), xi


def _tq1_byte(digits: np.ndarray) -> np.ndarray:
    """digits [..., n] most significant first -> ceil(q * 256 / 243) with q = sum digit * 3^(4 - i) (n = 4: times 3)."""
    q = np.zeros(digits.shape[:-1], np.int64)
    for i in range(digits.shape[-1]):
        q = q * 3 + digits[..., i]
    if digits.shape[-1] == 4:
        q = q * 3
    return ((q * 256 + 242) // 243).astype(np.uint8)


def gguf_quantize(values: np.ndarray, qtype: str) -> np.ndarray:
    """[N, K] float32 -> uint8 [N, K / 256 * block bytes] of TQ1_0 / TQ2_0 blocks (quantize_row_tq{1,2}_0_ref)."""
    d, xi = _gguf_digits(values)
    N, nb = d.shape
    dbytes = d.view(np.uint8).reshape(N, nb, 2)
    if qtype == "tq2_0":
        # two chunks of 128 elements: byte m of a chunk holds elements m, m + 32, m + 64, m + 96 at bits 0, 2, 4, 6
        c = xi.reshape(N, nb, 2, 4, 32)
        qs = (c[:, :, :, 0] | (c[:, :, :, 1] << 2) | (c[:, :, :, 2] << 4) | (c[:, :, :, 3] << 6)).astype(np.uint8).reshape(N, nb, 64)
        return np.concatenate([qs, dbytes], -1).reshape(N, nb * GGUF_TQ2_0_BYTES)
    if qtype == "tq1_0":
        a = xi[:, :, :160].reshape(N, nb, 5, 32)          # element m + 32 n -> byte m, digit n
        b = xi[:, :, 160:240].reshape(N, nb, 5, 16)       # element 160 + m + 16 n -> byte 32 + m, digit n
        h = xi[:, :, 240:].reshape(N, nb, 4, 4)           # element 240 + j + 4 m -> qh[j], digit m
        qs = np.concatenate([_tq1_byte(np.moveaxis(a, 2, -1)), _tq1_byte(np.moveaxis(b, 2, -1))], -1)
        qh = _tq1_byte(np.moveaxis(h, 2, -1))
        return np.concatenate([qs, qh, dbytes], -1).reshape(N, nb * GGUF_TQ1_0_BYTES)
    raise ValueError(f"unknown ggml type {qtype!r}")


def gguf_dequantize(blocks: np.ndarray, qtype: str, K: int) -> np.ndarray:
    """uint8 blocks [N, ...] -> float32 [N, K] (dequantize_row_tq{1,2}_0): (digit - 1) * d."""
    blocks = np.asarray(blocks, np.uint8)
    N = blocks.shape[0]
    nb = K // GGUF_QK
    if qtype == "tq2_0":
        b = blocks.reshape(N, nb, GGUF_TQ2_0_BYTES)
        qs = b[:, :, :64].reshape(N, nb, 2, 1, 32).astype(np.int64)
        dig = (qs >> (2 * np.arange(4)).reshape(1, 1, 1, 4, 1)) & 3
        d = np.ascontiguousarray(b[:, :, 64:]).view(np.float16).reshape(N, nb).astype(np.float32)
        return ((dig.reshape(N, nb, GGUF_QK) - 1).astype(np.float32) * d[..., None]).reshape(N, K)
    if qtype == "tq1_0":
        b = blocks.reshape(N, nb, GGUF_TQ1_0_BYTES)
        pow3 = np.array([1, 3, 9, 27, 81], np.int64)

        def digits(q, n):  # digit i (most significant first) of each byte: ((q * 3^i mod 256) * 3) >> 8
            qq = (q.astype(np.int64)[..., None, :] * pow3[:n].reshape(-1, 1)) & 0xFF
            return (qq * 3) >> 8

        a = digits(b[:, :, :32], 5).reshape(N, nb, 160)
        c = digits(b[:, :, 32:48], 5).reshape(N, nb, 80)
        h = digits(b[:, :, 48:52], 4).reshape(N, nb, 16)
        d = np.ascontiguousarray(b[:, :, 52:]).view(np.float16).reshape(N, nb).astype(np.float32)
        dig = np.concatenate([a, c, h], -1)
        return ((dig - 1).astype(np.float32) * d[..., None]).reshape(N, K)
    raise ValueError(f"unknown ggml type {qtype!r}")

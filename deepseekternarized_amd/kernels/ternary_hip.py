"""Ternary GEMM and grouped (MoE expert) GEMM on gfx950: the kernel backend interface.

Mirror of ``boilerplate/kernels/ternary_cuda.py`` (names, argument meaning, error behaviour); the
contract is the reference's::

    out[t, n] = x_scale[t] * sum_g w_scale[e(t), n, g] * sum_{k in g} x[t, k] * trit[e(t), n, k]

Every function launches HIP kernels from ``libbp_ternary_hip.so``; nothing is computed in Python or
on the CPU. Where the reference falls back to a PyTorch or C++ CPU path (CPU tensors, missing
extension) this module raises instead.

Additions behind the same API: float activations (bf16/f16/f32, ``x_scale=None``), scales in their
stored dtype (fp16/bf16) as well as float32, and several stacked terms per call (pass lists of
``packed`` / ``w_scale`` tensors) summed in one pass over the activations.
"""

from __future__ import annotations

import ctypes as C
import os
from functools import lru_cache

import torch

from . import _lib

_BACKENDS = ("auto", "cuda", "hip", "torch", "cpp")


_WORKSPACE_CAP = 8 << 30  # bytes of workspace the mirrored grouped call allocates at most
_DECODE_ROWS = 6  # bf16 / int8 calls of up to this many rows per expert run on the decode kernels: no workspace query


class _HipTernary:
    """Object returned by :func:`ext`: the native module surface of the reference
    (``boilerplate/kernels/csrc/ternary_cuda.cpp:7-10``) over the C ABI."""

    def __init__(self, lib):
        self.lib = lib

    def ternary_grouped_gemm(self, out, x, x_scale, offsets, packed, w_scale, K, group, fmt, lut1=None, max_rows=None,
                             offsets_host=None):
        """``out`` [T, N] f32 is accumulated into. Positional arguments as in
        ``ternary_cuda_kernel.cu:103-108``; ``packed`` / ``w_scale`` may be lists (stacked terms)."""
        packed_l = list(packed) if isinstance(packed, (list, tuple)) else [packed]
        scale_l = list(w_scale) if isinstance(w_scale, (list, tuple)) else [w_scale]
        if len(packed_l) != len(scale_l) or not 1 <= len(packed_l) <= _lib.BP_MAX_TERMS:
            raise RuntimeError("packed and w_scale must hold the same number of terms (1..4)")
        tensors = [out, x, offsets, *packed_l, *scale_l] + ([x_scale] if x_scale is not None else [])
        for t in tensors:
            if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous()):
                raise RuntimeError("ternary GEMM tensors must be contiguous HIP device tensors")
            if t.device != out.device:
                raise RuntimeError("ternary GEMM tensors must share one device")
        if out.dtype != torch.float32 or offsets.dtype != torch.int64 or any(p.dtype != torch.uint8 for p in packed_l):
            raise RuntimeError("unexpected ternary GEMM dtype")
        if x_scale is not None and x_scale.dtype != torch.float32:
            raise RuntimeError("unexpected ternary GEMM dtype (x_scale must be float32)")
        if x.dtype == torch.int8 and x_scale is None:
            raise RuntimeError("int8 activations need x_scale")
        if any(p.dim() != 3 for p in packed_l) or any(s.dim() != 3 for s in scale_l) or x.dim() != 2 or out.dim() != 2:
            raise RuntimeError("bad ranks")
        E, N, Kp = packed_l[0].shape
        G = scale_l[0].shape[2]
        sdt = scale_l[0].dtype
        for p, s in zip(packed_l, scale_l):
            if tuple(p.shape) != (E, N, Kp) or tuple(s.shape) != (E, N, G) or s.dtype != sdt:
                raise RuntimeError("inconsistent ternary GEMM shapes")
        T = x.shape[0]
        if x.shape[1] != K or offsets.dim() != 1 or offsets.numel() != E + 1:
            raise RuntimeError("inconsistent ternary GEMM shapes")
        if tuple(out.shape) != (T, N) or (x_scale is not None and x_scale.numel() != T):
            raise RuntimeError("bad output shape")
        if lut1 is not None and lut1.numel() < 256 * 5:
            raise RuntimeError("inconsistent ternary GEMM shapes (lut1)")
        if max_rows is None:
            max_rows = T
        host = None
        if offsets_host is not None:
            host_t = torch.as_tensor(offsets_host, dtype=torch.int64).cpu().contiguous()
            if host_t.numel() != E + 1:
                raise RuntimeError("inconsistent ternary GEMM shapes (offsets)")
            host = host_t.data_ptr()
        pk = (C.c_void_p * len(packed_l))(*[p.data_ptr() for p in packed_l])
        sc = (C.c_void_p * len(scale_l))(*[s.data_ptr() for s in scale_l])
        dev = out.device
        xdt, index = _lib.dtype_code(x.dtype), dev.index if dev.index is not None else torch.cuda.current_device()
        switch = torch.cuda.current_device() != index  # (entering a device context costs microseconds: only when it changes anything)
        if switch:
            prev = torch.cuda.current_device()
            torch.cuda.set_device(index)
        try:
            stream = torch._C._cuda_getCurrentRawStream(index)
            # Prefill-sized calls get a workspace (the library allocates nothing itself): with one, the grouped GEMM kernels
            # for bf16 activations convert the activations once instead of once per block of output rows, and float32 /
            # fp16 activations run on the bf16 kernels as a pair. The size query answers 0 where the launch would not use
            # one (small calls, a loose max_rows); decode-sized bf16 / int8 calls never do and skip the query.
            need = 0
            if max_rows > _DECODE_ROWS or xdt in (_lib.BP_F16, _lib.BP_F32):
                need = self.lib.bp_grouped_gemm_workspace_bytes(xdt, T, N, int(K), E, int(fmt), int(max_rows))
                if need > _WORKSPACE_CAP:  # (about 2.1 bytes per activation: a call this large keeps its memory and runs the kernels without one)
                    need = 0
            head = (out.data_ptr(), x.data_ptr(), xdt, x_scale.data_ptr() if x_scale is not None else None, offsets.data_ptr(), host,
                    C.cast(pk, C.c_void_p), C.cast(sc, C.c_void_p), _lib.dtype_code(sdt), len(packed_l),
                    T, N, int(K), Kp, G, int(group), E, int(fmt), int(max_rows))
            if need:
                ws = torch.empty(need, dtype=torch.uint8, device=dev)
                rc = self.lib.bp_ternary_grouped_gemm_ws(*head, ws.data_ptr(), need, stream)
            else:
                rc = self.lib.bp_ternary_grouped_gemm(*head, lut1.data_ptr() if lut1 is not None else None, stream)
        finally:
            if switch:
                torch.cuda.set_device(prev)
        if rc:
            _lib.check(rc)

    def last_kernel(self) -> str:
        return self.lib.bp_last_kernel().decode()

    def set_kernel_policy(self, policy: int) -> int:
        return self.lib.bp_set_kernel_policy(int(policy))


@lru_cache(1)
def ext():
    """The native module, or ``None`` when there is no HIP device (``boilerplate/kernels/ternary_cuda.py:32-43``
    tests ``torch.version.cuda``; on ROCm the toolkit shows up as ``torch.version.hip``).
    ``BOILERPLATE_NO_CUDA=1`` disables it as in the reference. With a device present the library
    must exist: a missing build raises instead of silently disabling the backend."""
    if os.environ.get("BOILERPLATE_NO_CUDA") or torch.version.hip is None or not torch.cuda.is_available():
        return None
    return _HipTernary(_lib.load())


def _fmt_code(fmt: str) -> int:
    """boilerplate/kernels/ternary_cuda.py:46-49."""
    if fmt not in ("tq1", "tq2"):
        raise ValueError(f"unknown ternary packing {fmt!r}")
    return 2 if fmt == "tq2" else 1


def _need_ext(x):
    e = ext()
    if e is None or not x.is_cuda:
        raise RuntimeError("HIP ternary kernel unavailable (no GPU, tensors not on a HIP device, or "
                           "BOILERPLATE_NO_CUDA); this build has no CPU fallback")
    return e


_dense_offsets_cache: dict = {}


def dense_offsets(device, rows: int) -> torch.Tensor:
    """The device offsets ``[0, rows]`` of a one-expert (dense) call, made once per device and row count and kept:
    a dense linear then costs no host-to-device copy per call."""
    key = (device, rows)
    t = _dense_offsets_cache.get(key)
    if t is None:
        if len(_dense_offsets_cache) > 4096:
            _dense_offsets_cache.clear()
        t = torch.tensor([0, rows], dtype=torch.int64, device=device)
        _dense_offsets_cache[key] = t
    return t


def _as_terms(packed, w_scale):
    pk = list(packed) if isinstance(packed, (list, tuple)) else [packed]
    sc = list(w_scale) if isinstance(w_scale, (list, tuple)) else [w_scale]
    return pk, sc


def ternary_gemm(x: torch.Tensor, x_scale: torch.Tensor, packed, w_scale, K: int, group: int, fmt: str,
                 backend: str = "auto") -> torch.Tensor:
    """[T, K] int8 activations x [N, Kp] packed weights -> [T, N] float32
    (``boilerplate/kernels/ternary_cuda.py:67-87``). ``backend="torch"`` selects the kernel that
    follows the reference's operation order exactly (:func:`ternary_gemm_ref`)."""
    _fmt_code(fmt)
    if x.dtype != torch.int8:
        raise TypeError("ternary_gemm takes int8 activations (see quant_act_int8)")
    pk, sc = _as_terms(packed, w_scale)
    _need_ext(x)
    return grouped_ternary_gemm(x, x_scale, dense_offsets(x.device, x.size(0)), [p[None] for p in pk], [s[None] for s in sc], K, group,
                                fmt, backend=backend, max_rows=x.size(0))


def ternary_gemm_float(x: torch.Tensor, packed, w_scale, K: int, group: int, fmt: str,
                       backend: str = "auto") -> torch.Tensor:
    """Float-activation product (the contract of the CPU kernel's float path,
    ``boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77,114-124``): x bf16/f16/f32 [T, K] -> [T, N] float32."""
    _fmt_code(fmt)
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError("ternary_gemm_float takes bf16, f16 or f32 activations")
    pk, sc = _as_terms(packed, w_scale)
    _need_ext(x)
    return grouped_ternary_gemm(x, None, dense_offsets(x.device, x.size(0)), [p[None] for p in pk], [s[None] for s in sc], K, group, fmt,
                                backend=backend, max_rows=x.size(0))


def ternary_gemm_ref(x: torch.Tensor, x_scale: torch.Tensor, packed: torch.Tensor, w_scale: torch.Tensor,
                     K: int, group: int, fmt: str) -> torch.Tensor:
    """The reference-order kernel: exact integer group sums, then float32 ``out += acc * w_scale[:, g]``
    in ascending g with separately rounded multiply and add, then ``* x_scale``
    (``boilerplate/kernels/ternary_cuda.py:52-64``), computed on the device."""
    return ternary_gemm(x, x_scale, packed, w_scale, K, group, fmt, backend="torch")


def grouped_ternary_gemm(x: torch.Tensor, x_scale, offsets, packed, w_scale, K: int, group: int, fmt: str,
                         backend: str = "auto", max_rows: int | None = None, validate: bool = False) -> torch.Tensor:
    """Rows of ``x`` sorted by expert; ``packed`` [E, N, Kp], ``w_scale`` [E, N, G] -> [T, N] float32
    (``boilerplate/kernels/ternary_cuda.py:90-111``).

    ``offsets`` given as host data (list, CPU tensor) is validated like the reference does and a
    violation raises ``ValueError("offsets ...")``. ``offsets`` given as a device tensor is used as is,
    with no device-to-host copy; the kernels clamp it, so it cannot cause out-of-bounds accesses.
    The launch then covers ``max_rows`` rows per expert - an upper bound the caller knows (the token count,
    when every token picks distinct experts), by default the row count of ``x``; rows of an expert beyond
    ``max_rows`` would not be computed. With host offsets the widest expert is taken from them and ``max_rows``
    is ignored. ``validate=True`` checks a caller's bound against device offsets on the device and raises the
    reference's error ("max_rows is smaller than the largest expert row count"); it reads one flag back, so it
    synchronises - a debugging aid, not for the serving path.
    """
    code = _fmt_code(fmt)
    if backend not in _BACKENDS:
        raise ValueError(f"unknown backend {backend!r}")
    pk, sc = _as_terms(packed, w_scale)
    E = pk[0].size(0)
    on_device = isinstance(offsets, torch.Tensor) and offsets.is_cuda
    host = None
    if not on_device:
        host = torch.as_tensor(offsets, dtype=torch.int64).cpu()
        if host.numel() != E + 1 or int(host[0]) != 0 or int(host[-1]) != x.size(0) or bool((host.diff() < 0).any()):
            raise ValueError("offsets must be nondecreasing, start at 0, end at the row count, one per expert + 1")
    if backend == "cpp":
        raise RuntimeError("C++ CPU ternary kernel unavailable in this build (HIP kernels only)")
    e = _need_ext(x)
    dev = x.device
    offs_dev = offsets.to(torch.int64).contiguous() if on_device else host.to(dev, non_blocking=False)
    if host is not None:
        max_rows = int(host.diff().max()) if E else 0
    elif max_rows is None:
        max_rows = x.size(0)
    else:
        max_rows = max(0, min(int(max_rows), x.size(0)))
    if validate and on_device and E:
        flag = torch.zeros(1, dtype=torch.int32, device=dev)
        with torch.cuda.device(dev):
            _lib.check(e.lib.bp_check_max_rows(flag.data_ptr(), offs_dev.data_ptr(), E, x.size(0), max_rows, _lib.stream_ptr(dev)))
        if int(flag):
            raise RuntimeError("max_rows is smaller than the largest expert row count")
    out = torch.zeros(x.size(0), pk[0].size(1), dtype=torch.float32, device=dev)
    xs = None if x_scale is None else x_scale.float().contiguous()
    args = (out, x.contiguous(), xs, offs_dev, [p.contiguous() for p in pk], [s.contiguous() for s in sc], K, group, code, None, max_rows)
    if backend != "torch":  # (the kernel policy is per thread and 0 unless someone changed it: nothing to set or restore)
        e.ternary_grouped_gemm(*args, offsets_host=host)
        return out
    old = e.set_kernel_policy(1)
    try:
        e.ternary_grouped_gemm(*args, offsets_host=host)
    finally:
        e.set_kernel_policy(old)
    return out


def sort_by_expert(expert_ids: torch.Tensor, n_experts: int, validate: bool = False) -> tuple[torch.Tensor, torch.Tensor]:
    """Flattened top-k expert ids [T*k] -> (row order sorting them by expert, offsets [E + 1])
    (``boilerplate/kernels/ternary_cuda.py:114-118``): a stable counting sort on the device.
    The result stays on the device; no host synchronisation happens.

    Ids outside ``[0, n_experts)`` - which the reference's ``bincount`` / ``argsort`` reject or sort to the ends - are
    left out of the count: ``offsets[-1]`` is then smaller than the number of ids and the tail of ``order`` holds -1.
    ``validate=True`` reads a device flag back (one host synchronisation) and raises ValueError for such ids instead."""
    e = _need_ext(expert_ids)
    ids = expert_ids.to(torch.int64).contiguous().view(-1)
    n, dev = ids.numel(), ids.device
    order = torch.full((n,), -1, dtype=torch.int64, device=dev) if validate else torch.empty(n, dtype=torch.int64, device=dev)
    offsets = torch.empty(n_experts + 1, dtype=torch.int64, device=dev)
    need = e.lib.bp_sort_workspace_ints(n, n_experts)
    ws = torch.empty(need, dtype=torch.int32, device=dev) if need else None
    bad = torch.zeros(1, dtype=torch.int32, device=dev) if validate else None
    with torch.cuda.device(dev):
        _lib.check(e.lib.bp_sort_by_expert(order.data_ptr(), offsets.data_ptr(), ids.data_ptr(), n, n_experts,
                                           ws.data_ptr() if ws is not None else None,
                                           bad.data_ptr() if bad is not None else None, _lib.stream_ptr(dev)))
    if validate and int(bad.item()):
        raise ValueError(f"expert ids must lie in [0, {n_experts})")
    return order, offsets


def gather_rows(src: torch.Tensor, index: torch.Tensor, divisor: int = 1) -> torch.Tensor:
    """``src[index // divisor]`` for a 2-D ``src``: the token-to-expert permute
    (``scripts/eval/ternary_kernel_bench.py:90-93``) as one device kernel."""
    e = _need_ext(src)
    src = src.contiguous()
    index = index.to(torch.int64).contiguous()
    rows, row_bytes = index.numel(), src.size(1) * src.element_size()
    if row_bytes % 2:
        raise RuntimeError("gather_rows needs an even number of bytes per row")
    dst = torch.empty(rows, src.size(1), dtype=src.dtype, device=src.device)
    with torch.cuda.device(src.device):
        _lib.check(e.lib.bp_gather_rows(dst.data_ptr(), src.data_ptr(), index.data_ptr(), int(divisor), rows,
                                        src.size(0), row_bytes, _lib.stream_ptr(src.device)))
    return dst

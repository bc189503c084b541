"""Routed-expert MoE layer on the grouped ternary GEMM.

The reference engines run a MoE layer as a Python loop over all experts with one ``TernaryLinear`` call
per projection (``boilerplate/engine/standard.py:151-176``; the grouped kernel API is not wired into
them). This module runs the same computation, with the same rounding points, as one sort of the routing,
one row gather and three grouped launches (gate and up share one launch over a stacked [E, 2I, Kp]
weight):

    scores = softmax(router_logits.float()); values, indices = topk(scores, k); values -> x.dtype
    per (token, slot): y = down(silu(gate(x)) * up(x)) * value, each linear rounded to x.dtype,
    out[token] += y in ascending expert order, accumulated in x.dtype

softmax / topk are torch ops (as in the reference); everything touching packed weights runs in the HIP
kernels. bf16 activations (``act="bf16"``) or per-row int8 (``act="int8"``, Mode D default).

``pattern="v4"`` runs the rounding points of the V4 engine instead (``boilerplate/engine/model.py:376-387`` ``swiglu``,
``:407-422`` ``moe``): the caller's router hands over float32 weights and expert ids, gate / up are rounded to bf16 and
widened again, clamped by ``swiglu_limit``, ``weights * (silu(gate) * up)`` is float32 and rounded once as the input of
the down projection, and a token's experts are added in float32 in ascending expert order.
"""

from __future__ import annotations

import torch

from .kernels import _lib
from .kernels.ternary_hip import _fmt_code, _need_ext, gather_rows, grouped_ternary_gemm, sort_by_expert
from .ternary.ops import quant_act_int8


def swiglu_bf16(gate_up: torch.Tensor, inter: int) -> torch.Tensor:
    """bf16(bf16(silu(bf16 gate)) * bf16 up) from a float32 [rows, 2 * inter] gate|up product
    (``StandardDecoder._run_mlp``, boilerplate/engine/standard.py:151-154, on bf16 tensors)."""
    e = _need_ext(gate_up)
    rows = gate_up.size(0)
    h = torch.empty(rows, inter, dtype=torch.bfloat16, device=gate_up.device)
    up = gate_up[:, inter:]
    with torch.cuda.device(gate_up.device):
        _lib.check(e.lib.bp_swiglu_bf16(h.data_ptr(), gate_up.data_ptr(), up.data_ptr(), rows, inter, gate_up.stride(0),
                                        _lib.stream_ptr(gate_up.device)))
    return h


def moe_combine_bf16(y: torch.Tensor, inv: torch.Tensor, values: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
    """out[t] = sum over the token's slots, in ascending expert order, of bf16(bf16(y[inv[t, s]]) * values[t, s]),
    accumulated in bf16 (``output.index_add_`` on a bf16 tensor, boilerplate/engine/standard.py:173-175)."""
    e = _need_ext(y)
    T, k = indices.shape
    H = y.size(1)
    out = torch.empty(T, H, dtype=torch.bfloat16, device=y.device)
    with torch.cuda.device(y.device):
        _lib.check(e.lib.bp_moe_combine_bf16(out.data_ptr(), y.data_ptr(), inv.data_ptr(), values.data_ptr(),
                                             indices.data_ptr(), T, k, H, _lib.stream_ptr(y.device)))
    return out


class TernaryMoE:
    """``experts``: per projection a list of stacked terms ``(packed [E, N, Kp] uint8, scale [E, N, G])``:
    ``gate`` / ``up`` with N = inter, K = hidden; ``down`` with N = hidden, K = inter."""

    def __init__(self, gate, up, down, hidden: int, inter: int, top_k: int, fmt: str, group: int,
                 act: str = "bf16", renorm: bool = False, pattern: str = "standard", swiglu_limit: float = 0.0):
        _fmt_code(fmt)
        if act not in ("bf16", "int8"):
            raise ValueError(f"unknown activation mode {act!r}")
        if pattern not in ("standard", "v4"):
            raise ValueError(f"unknown MoE call pattern {pattern!r}")
        if not swiglu_limit >= 0.0:
            raise ValueError("swiglu_limit must be 0 (no clamp) or positive")
        self.pattern, self.swiglu_limit = pattern, float(swiglu_limit)
        if not (len(gate) == len(up) == len(down)):
            raise ValueError("gate, up and down must hold the same number of stacked terms")
        self.hidden, self.inter, self.top_k, self.fmt, self.group, self.act, self.renorm = hidden, inter, top_k, fmt, group, act, renorm
        self.n_experts = gate[0][0].size(0)
        # gate and up stacked along N once, so both projections of an expert stream in one launch
        self.gate_up = [(torch.cat([g[0], u[0]], 1).contiguous(), torch.cat([g[1], u[1]], 1).contiguous())
                        for g, u in zip(gate, up)]
        self.down = [(p.contiguous(), s.contiguous()) for p, s in down]

    def _linear(self, x, terms, K):
        if self.act == "int8":
            q, s = quant_act_int8(x)
        else:
            q, s = x, None
        return grouped_ternary_gemm(q, s, self._offsets, [p for p, _ in terms], [sc for _, sc in terms], K, self.group, self.fmt,
                                    max_rows=self._max_rows)

    def route(self, router_logits: torch.Tensor, tokens: int):
        """``softmax`` / ``topk`` of the router logits (engine/standard.py:160-165): routing weights bf16 [T, k], expert
        ids int64 [T, k], slots in descending score. One launch (``bp_route_topk``: float32 softmax, ties to the lower
        expert id) for up to 1024 experts; beyond, the same torch ops the reference uses."""
        logits = router_logits.reshape(tokens, -1)
        E = logits.size(-1)
        if E <= 1024 and self.top_k <= min(E, 64) and logits.dtype in (torch.bfloat16, torch.float16, torch.float32):
            e = _need_ext(logits)
            logits = logits.contiguous()
            values = torch.empty(tokens, self.top_k, dtype=torch.bfloat16, device=logits.device)
            indices = torch.empty(tokens, self.top_k, dtype=torch.int64, device=logits.device)
            with torch.cuda.device(logits.device):
                _lib.check(e.lib.bp_route_topk(values.data_ptr(), _lib.BP_BF16, indices.data_ptr(), logits.data_ptr(), _lib.dtype_code(logits.dtype),
                                               tokens, E, self.top_k, int(self.renorm), _lib.stream_ptr(logits.device)))
            return values, indices
        scores = torch.softmax(logits.float(), dim=-1)
        values, indices = torch.topk(scores, self.top_k, dim=-1)
        if self.renorm:
            values = values / values.sum(-1, keepdim=True)
        return values.to(torch.bfloat16).contiguous(), indices.contiguous()

    def _workspace(self, tokens: int, device) -> torch.Tensor:
        e = _need_ext(self.down[0][0])
        need = int(e.lib.bp_moe_layer_workspace_bytes(tokens, self.hidden, self.inter, self.n_experts, self.top_k,
                                                      _lib.BP_I8 if self.act == "int8" else _lib.BP_BF16, _fmt_code(self.fmt)))
        device = torch.device(device)
        if device.index is None:  # torch.device("cuda") != torch.device("cuda:0"): compare devices with their index
            device = torch.device(device.type, torch.cuda.current_device())
        ws = getattr(self, "_ws", None)
        if ws is None or ws.numel() < need or ws.device != device:
            # A HIP graph captured by graphed() holds the address of the workspace it ran in: a workspace that is
            # replaced stays referenced (self._ws_captured) instead of going back to the allocator under that graph.
            if ws is not None and getattr(self, "_ws_in_graph", False):
                self.__dict__.setdefault("_ws_captured", []).append(ws)
                self._ws_in_graph = False
            self._ws = ws = torch.empty(need, dtype=torch.uint8, device=device)   # (reused by later calls of up to this many tokens)
        return ws

    def __call__(self, x: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        """The layer through ``bp_moe_layer_bf16``: one library call after the router's top-k, no host synchronisation
        (the grouped launches take the token tiles from a device-side list), intermediates in a cached workspace."""
        shape = x.shape
        flat = x.reshape(-1, self.hidden).to(torch.bfloat16).contiguous()
        e = _need_ext(flat)
        T = flat.size(0)
        if self.pattern == "v4":
            raise RuntimeError('a pattern="v4" layer takes the router\'s output: call routed(x, weights, indices)')
        values, indices = self.route(router_logits, T)
        out = torch.empty(T, self.hidden, dtype=torch.bfloat16, device=flat.device)
        if T == 0:
            return out.view(shape).to(x.dtype)
        self._launch(e, out, flat, values, indices, T)
        return out.view(shape).to(x.dtype)

    def _launch(self, e, out, flat, values, indices, T, out_dtype=None):
        import ctypes as C

        ws = self._workspace(T, flat.device)
        if torch.cuda.is_current_stream_capturing():
            self._ws_in_graph = True
        n = len(self.down)
        arr = lambda ts: (C.c_void_p * n)(*[t.data_ptr() for t in ts])
        gp, gs = arr([p for p, _ in self.gate_up]), arr([s for _, s in self.gate_up])
        dp, ds = arr([p for p, _ in self.down]), arr([s for _, s in self.down])
        sdt = {torch.float32: _lib.BP_F32, torch.float16: _lib.BP_F16, torch.bfloat16: _lib.BP_BF16}[self.down[0][1].dtype]
        tail = (gp, gs, dp, ds, sdt, n, T, self.hidden, self.inter, self.n_experts, self.top_k, self.group, _fmt_code(self.fmt),
                _lib.BP_I8 if self.act == "int8" else _lib.BP_BF16, ws.data_ptr(), ws.numel(), None, _lib.stream_ptr(flat.device))
        with torch.cuda.device(flat.device):
            if self.pattern == "v4":
                _lib.check(e.lib.bp_moe_layer_v4(out.data_ptr(), out_dtype, flat.data_ptr(), indices.data_ptr(), values.data_ptr(),
                                                 self.swiglu_limit, *tail))
            else:
                _lib.check(e.lib.bp_moe_layer_bf16(out.data_ptr(), flat.data_ptr(), indices.data_ptr(), values.data_ptr(), *tail))

    def routed(self, x: torch.Tensor, weights: torch.Tensor, indices: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
        """The routed experts of a V4 layer (``pattern="v4"``) through ``bp_moe_layer_v4``: ``weights`` float32 [T, k] and
        ``indices`` int64 [T, k] are the router's output (boilerplate/engine/model.py:389-405 stays with the caller, as do the
        shared experts). Returns the float32 sum ``y`` of model.py:411-420 (``out_dtype=torch.float32``: the caller adds
        its shared experts and casts, :421-422) or that sum cast once to bf16."""
        if self.pattern != "v4":
            raise RuntimeError('routed() is the entry of pattern="v4" layers')
        if out_dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("out_dtype must be torch.float32 or torch.bfloat16")
        shape = x.shape
        flat = x.reshape(-1, self.hidden).to(torch.bfloat16).contiguous()
        e = _need_ext(flat)
        T = flat.size(0)
        w = weights.reshape(T, self.top_k).to(torch.float32).contiguous()
        idx = indices.reshape(T, self.top_k).to(torch.int64).contiguous()
        out = torch.empty(T, self.hidden, dtype=out_dtype, device=flat.device)
        if T:
            self._launch(e, out, flat, w, idx, T, _lib.dtype_code(out_dtype))
        return out.view(shape)

    def composed(self, x: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
        """The same layer as separate library calls (sort, gather, two grouped GEMMs, SwiGLU, combine), sizing the
        grouped launches the reference's way: beyond 64 tokens the widest expert's row count is read back to the host
        (boilerplate/kernels/ternary_cuda.py:97). Kept as the check of ``__call__`` and for callers that want the stages."""
        if self.pattern != "standard":
            raise RuntimeError("composed() restates the standard decoder's layer only")
        shape = x.shape
        flat = x.reshape(-1, self.hidden).to(torch.bfloat16).contiguous()
        _need_ext(flat)
        values, indices = self.route(router_logits, flat.size(0))
        order, self._offsets = sort_by_expert(indices.reshape(-1), self.n_experts)
        # Rows of the widest expert: at most one per token (top-k picks distinct experts). For a few tokens that
        # bound costs nothing and keeps the layer free of host synchronisation; for many, the launch would cover
        # tiles that do not exist, so the exact figure is read back, as the reference does
        # (boilerplate/kernels/ternary_cuda.py:97, `int(offs.diff().max())`).
        T = flat.size(0)
        self._max_rows = T if T <= 64 else int((self._offsets[1:] - self._offsets[:-1]).max())
        inv = torch.empty_like(order)
        inv[order] = torch.arange(order.numel(), device=order.device)
        xg = gather_rows(flat, order, self.top_k)                                  # [T*k, H] rows in expert order
        gu = self._linear(xg, self.gate_up, self.hidden)                           # f32 [T*k, 2I]
        h = swiglu_bf16(gu, self.inter)                                            # bf16 [T*k, I]
        y = self._linear(h, self.down, self.inter)                                 # f32 [T*k, H]
        out = moe_combine_bf16(y, inv, values, indices)
        return out.view(shape).to(x.dtype)

    def graphed(self, tokens: int, dtype: torch.dtype = torch.bfloat16, device="cuda"):
        """The layer for a fixed number of tokens as one HIP graph: ``run(x [tokens, hidden], router_logits [tokens, E])``
        copies its arguments into the graph's input buffers, replays the captured launches and returns the graph's
        output buffer (overwritten by the next replay). With a handful of tokens the layer is a dozen launches of a few
        microseconds each, and issuing them costs more than running them; a replay issues them at once.
        Any number of tokens: the layer never reads the routing back to the host."""
        if tokens < 1:
            raise ValueError("graphed() needs at least one token")
        if self.pattern != "standard":
            raise RuntimeError("graphed() captures the standard decoder's layer")
        self._workspace(tokens, device)
        xs = torch.zeros(tokens, self.hidden, dtype=dtype, device=device)
        ls = torch.zeros(tokens, self.n_experts, dtype=torch.float32, device=device)
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):  # warm-up outside the capture: kernel attributes, lazy module loads, allocator state
            for _ in range(2):
                self(xs, ls)
        torch.cuda.current_stream(device).wait_stream(side)
        torch.cuda.synchronize(device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = self(xs, ls)

        def run(x: torch.Tensor, router_logits: torch.Tensor) -> torch.Tensor:
            xs.copy_(x.reshape(tokens, self.hidden))
            ls.copy_(router_logits.reshape(tokens, self.n_experts))
            graph.replay()
            return out

        run.graph = graph  # keeps the graph (and its memory pool) alive with the callable
        run.workspace = self._ws  # ... and the workspace whose address the captured launches hold
        return run


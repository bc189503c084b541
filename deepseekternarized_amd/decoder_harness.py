"""Random-init OLMoE-shaped Mode D decoder used to time the ternary path end to end.

This is the measurement harness for the reference's ``boilerplate bench`` loop
(``boilerplate/cli.py:145-224``: warm-up, timed prefill of ``[batch, prompt]`` ids, then ``gen`` greedy
decode steps with a concatenated KV cache) on a ``StandardDecoder``-shaped model
(``boilerplate/engine/standard.py:178-227``): per layer RMSNorm -> q/k/v ternary linears -> RoPE ->
causal attention -> o ternary linear -> RMSNorm -> routed-expert MoE. It is NOT a port of the engine:
there is no checkpoint/manifest loading, tokenizer or expert cache; weights are random ternary draws.
Every ternary linear and the MoE run through the HIP kernels; norms, RoPE, attention and the dense
embedding / router / head are torch ops, as they are in the reference.
"""

from __future__ import annotations

import math
import time
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from .moe import TernaryMoE
from .ternary.ops import PackedTerm, TernaryLinear
from .ternary.pack import pack


@dataclass
class DecoderConfig:
    layers: int = 16
    hidden: int = 2048
    heads: int = 16
    experts: int = 64
    top_k: int = 8
    inter: int = 1024
    vocab: int = 50304
    fmt: str = "tq2"
    group: int = 128
    act: str = "int8"  # Mode D default (boilerplate/qat/export.py:78-79)
    theta: float = 10000.0
    eps: float = 1e-5


def random_ternary(E, N, K, fmt, group, gen, scale_mean=0.02):
    """[E, N, Kp] packed trits (P(-1) = P(+1) = 0.33) and fp16 scales scale_mean * |N(0, 1)|."""
    packed = torch.empty(E, N, -(-K // (4 if fmt == "tq2" else 5)), dtype=torch.uint8, device="cuda")
    for e in range(E):
        u = torch.rand(N, K, device="cuda", generator=gen)
        packed[e] = pack(torch.where(u < 0.33, -1, torch.where(u < 0.66, 1, 0)).to(torch.int8), fmt)
    scale = (scale_mean * torch.randn(E, N, K // group, device="cuda", generator=gen).abs()).half()
    return packed, scale


class _Layer:
    pass


class TernaryDecoder:
    def __init__(self, cfg: DecoderConfig, seed: int = 0, dtype=torch.bfloat16):
        self.cfg, self.dtype = cfg, dtype
        g = torch.Generator(device="cuda").manual_seed(seed)
        H = cfg.hidden
        self.head_dim = H // cfg.heads
        s = 1.0 / math.sqrt(H)
        self.embedding = (torch.randn(cfg.vocab, H, device="cuda", generator=g) * 0.5).to(dtype)
        self.head = (torch.randn(cfg.vocab, H, device="cuda", generator=g) * s).to(dtype)
        self.final_norm = torch.ones(H, device="cuda", dtype=dtype)
        self.layers = []
        wscale = 1.5 * s  # keeps activations O(1) through the random layers
        for _ in range(cfg.layers):
            L = _Layer()
            L.input_norm = torch.ones(H, device="cuda", dtype=dtype)
            L.post_norm = torch.ones(H, device="cuda", dtype=dtype)
            # q | k | v stacked along N like the experts' gate | up: one activation quantisation and one launch for the three
            qkv = [random_ternary(1, H, H, cfg.fmt, cfg.group, g, wscale) for _ in range(3)]
            L.qkv = TernaryLinear([PackedTerm(torch.cat([p[0] for p, _ in qkv]), torch.cat([sc[0] for _, sc in qkv]))], H, cfg.fmt, cfg.group, act=cfg.act)
            p, sc = random_ternary(1, H, H, cfg.fmt, cfg.group, g, wscale)
            L.o = TernaryLinear([PackedTerm(p[0], sc[0])], H, cfg.fmt, cfg.group, act=cfg.act)
            L.router = (torch.randn(cfg.experts, H, device="cuda", generator=g) * s).to(dtype)
            gate = random_ternary(cfg.experts, cfg.inter, H, cfg.fmt, cfg.group, g, wscale)
            up = random_ternary(cfg.experts, cfg.inter, H, cfg.fmt, cfg.group, g, wscale)
            down = random_ternary(cfg.experts, H, cfg.inter, cfg.fmt, cfg.group, g, 1.5 / math.sqrt(cfg.inter))
            L.experts = (gate, up, down)
            L.moe = TernaryMoE([gate], [up], [down], H, cfg.inter, cfg.top_k, cfg.fmt, cfg.group, act=cfg.act)
            self.layers.append(L)

    def _norm(self, x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.cfg.eps)).to(x.dtype) * w

    def _rope(self, q, k, offset):
        pos = torch.arange(offset, offset + q.size(-2), dtype=torch.float32, device=q.device)
        inv = self.cfg.theta ** (-torch.arange(0, self.head_dim, 2, dtype=torch.float32, device=q.device) / self.head_dim)
        fr = torch.outer(pos, inv)
        ang = torch.cat((fr, fr), dim=-1)
        cos, sin = ang.cos().to(q.dtype)[None, None], ang.sin().to(q.dtype)[None, None]

        def rot(x):
            a, b = x.chunk(2, dim=-1)
            return torch.cat((-b, a), dim=-1)

        return q * cos + rot(q) * sin, k * cos + rot(k) * sin

    def linear(self, lin, x):
        return lin(x, out_dtype=x.dtype)

    def moe(self, layer, z):
        return layer.moe(z, F.linear(z, layer.router))

    @torch.inference_mode()
    def forward(self, ids: torch.Tensor, past=None):
        """ids [batch, seq] continuing ``past`` -> (float32 logits [batch, seq, vocab], new KV cache)."""
        past = [None] * len(self.layers) if past is None else past
        x = F.embedding(ids.cuda(), self.embedding).to(self.dtype)
        new_past = []
        for index, layer in enumerate(self.layers):
            residual = x
            z = self._norm(x, layer.input_norm)
            q, k, v = self.linear(layer.qkv, z).split(self.cfg.hidden, dim=-1)
            b, s, _ = q.shape
            q = q.view(b, s, self.cfg.heads, self.head_dim).transpose(1, 2)
            k = k.view(b, s, self.cfg.heads, self.head_dim).transpose(1, 2)
            v = v.view(b, s, self.cfg.heads, self.head_dim).transpose(1, 2)
            offset = 0 if past[index] is None else past[index][0].size(-2)
            q, k = self._rope(q, k, offset)
            if past[index] is not None:
                k = torch.cat((past[index][0], k), dim=-2)
                v = torch.cat((past[index][1], v), dim=-2)
            new_past.append((k, v))
            scores = (q @ k.transpose(-2, -1)) / math.sqrt(self.head_dim)
            mask = torch.arange(k.size(-2), device=x.device)[None, :] > torch.arange(offset, offset + s, device=x.device)[:, None]
            scores = scores.masked_fill(mask, torch.finfo(scores.dtype).min)
            attention = torch.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype) @ v
            x = residual + self.linear(layer.o, attention.transpose(1, 2).reshape(b, s, -1).contiguous())
            residual = x
            z = self._norm(x, layer.post_norm)
            x = residual + self.moe(layer, z)
        x = self._norm(x, self.final_norm)
        return F.linear(x, self.head).float(), new_past


class GraphedDecode:
    """Greedy decoding of one token per sequence as ONE HIP graph replay per step.

    A decode step of this model is about forty kernel launches per layer, each a few microseconds of device time, so
    issued one by one from Python the step is bound by the host. The step is therefore written with static shapes -
    a KV cache preallocated to ``max_len`` positions, the current length held in a device scalar, attention over all
    ``max_len`` positions with the unwritten ones masked - and captured once; ``step()`` replays it. Batches up to 64
    sequences (the routed-expert layer needs no host read-back up to there). The eager path (``forward`` with a
    concatenated cache, as the reference's engine does it) stays the reference for this one: same kernels, same
    rounding points; only the softmax rows are longer (masked tail), which can move its float32 sum by an ulp."""

    def __init__(self, model: TernaryDecoder, cache, max_len: int):
        cfg = model.cfg
        self.model, self.max_len = model, max_len
        b, h, n, d = cache[0][0].shape
        if not 1 <= b <= 64:
            raise ValueError("graphed decoding covers batches of 1..64 sequences")
        if n >= max_len:
            raise ValueError("max_len must exceed the cached length")
        dev = cache[0][0].device
        self.k = [torch.zeros(b, h, max_len, d, dtype=k.dtype, device=dev) for k, _ in cache]
        self.v = [torch.zeros(b, h, max_len, d, dtype=v.dtype, device=dev) for _, v in cache]
        for i, (k, v) in enumerate(cache):
            self.k[i][:, :, :n].copy_(k)
            self.v[i][:, :, :n].copy_(v)
        self.pos = torch.full((1,), n, dtype=torch.int64, device=dev)  # positions written so far = index of the next one
        self.ids = torch.zeros(b, dtype=torch.int64, device=dev)
        pos_all = torch.arange(max_len, dtype=torch.float32, device=dev)
        inv = cfg.theta ** (-torch.arange(0, model.head_dim, 2, dtype=torch.float32, device=dev) / model.head_dim)
        fr = torch.outer(pos_all, inv)
        ang = torch.cat((fr, fr), dim=-1)
        self.cos, self.sin = ang.cos().to(model.dtype), ang.sin().to(model.dtype)  # [max_len, head_dim]
        self.arange = torch.arange(max_len, device=dev)
        self.logits = None
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):  # warm-up outside the capture (kernel attributes, cached offsets, allocator state)
            saved = (self.pos.clone(), [k.clone() for k in self.k], [v.clone() for v in self.v])
            for _ in range(2):
                self._step()
            self.pos.copy_(saved[0])
            for i in range(len(self.k)):
                self.k[i].copy_(saved[1][i])
                self.v[i].copy_(saved[2][i])
            del saved
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.logits = self._step()

    @torch.inference_mode()
    def _step(self):
        m, cfg = self.model, self.model.cfg
        x = F.embedding(self.ids[:, None], m.embedding).to(m.dtype)  # [b, 1, H]
        cos, sin = self.cos.index_select(0, self.pos)[None, None], self.sin.index_select(0, self.pos)[None, None]
        mask = (self.arange > self.pos)[None, None, None, :]  # positions not written yet

        def rot(t):
            a, b = t.chunk(2, dim=-1)
            return torch.cat((-b, a), dim=-1)

        for index, layer in enumerate(m.layers):
            residual = x
            z = m._norm(x, layer.input_norm)
            q, k, v = m.linear(layer.qkv, z).split(m.cfg.hidden, dim=-1)
            b = q.size(0)
            q = q.view(b, 1, cfg.heads, m.head_dim).transpose(1, 2)
            k = k.view(b, 1, cfg.heads, m.head_dim).transpose(1, 2)
            v = v.view(b, 1, cfg.heads, m.head_dim).transpose(1, 2)
            q, k = q * cos + rot(q) * sin, k * cos + rot(k) * sin
            self.k[index].index_copy_(2, self.pos, k)
            self.v[index].index_copy_(2, self.pos, v)
            scores = (q @ self.k[index].transpose(-2, -1)) / math.sqrt(m.head_dim)
            scores = scores.masked_fill(mask, torch.finfo(scores.dtype).min)
            attention = torch.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype) @ self.v[index]
            x = residual + m.linear(layer.o, attention.transpose(1, 2).reshape(b, 1, -1).contiguous())
            residual = x
            z = m._norm(x, layer.post_norm)
            x = residual + m.moe(layer, z)
        x = m._norm(x, m.final_norm)
        logits = F.linear(x, m.head).float()[:, 0]
        self.pos.add_(1)
        return logits

    def step(self, ids: torch.Tensor) -> torch.Tensor:
        """ids [batch] (the tokens just chosen) -> float32 logits [batch, vocab] of the next position (the graph's
        output buffer: overwritten by the next step)."""
        self.ids.copy_(ids)
        self.graph.replay()
        return self.logits


def bench_decoder(model: TernaryDecoder, batch: int, prompt_len: int, gen_len: int, seed: int = 0, graph: bool = False) -> dict:
    """The timing loop of ``boilerplate bench`` (cli.py:161-184): 8-token warm-up, timed prefill, greedy decode.
    ``graph``: the decode steps as HIP graph replays (:class:`GraphedDecode`; capture is outside the timed region)."""
    g = torch.Generator().manual_seed(seed)
    prompts = torch.randint(0, model.cfg.vocab, (batch, prompt_len), generator=g)
    model.forward(prompts[:, :8])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits, cache = model.forward(prompts)
    torch.cuda.synchronize()
    t_pre = time.perf_counter() - t0
    nxt = logits[:, -1].argmax(-1)
    if graph:
        dec = GraphedDecode(model, cache, prompt_len + gen_len + 1)
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(gen_len):
        if graph:
            logits = dec.step(nxt)
            nxt = logits.argmax(-1)
        else:
            logits, cache = model.forward(nxt[:, None], cache)
            nxt = logits[:, -1].argmax(-1)
    torch.cuda.synchronize()
    t_dec = time.perf_counter() - t0
    return {"batch": batch, "prompt_len": prompt_len, "gen_len": gen_len, "decode_as_hip_graph": bool(graph),
            "prefill_tok_s": round(batch * prompt_len / t_pre, 2),
            "decode_tok_s": round(batch * gen_len / t_dec, 3) if gen_len else None,
            "prefill_s": round(t_pre, 4), "decode_s": round(t_dec, 4),
            "peak_vram_bytes": torch.cuda.max_memory_allocated(), "finite": bool(torch.isfinite(logits).all())}

"""Benchmark of the ternary expert-linear path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--spin-up SECONDS] [--workload NAME] [--no-extras] [--no-cpu]

A step is one pass of the hot path over one batch of synthetic input. For the decode workloads (the default is
the headline configuration: TQ1, K = 7168, N = 2048, one token, bf16) it is one grouped launch that streams L distinct packed
linears of the named configuration (L chosen so the packed weights exceed the 256 MB Infinity Cache, i.e. every step
reads its weights from HBM). `--workload cfg3_grouped` times the grouped-expert GEMM of config 3 (value in TFLOP/s,
roofline against the bf16 MFMA peak), `--workload cfg2_moe_T{1,32,256}` one routed-expert layer of config 2; these
single-workload runs are also what counter collection (rocprofv3 --pmc) is run on. Inputs are resident in HBM
before the timed region. Every timed launch sequence is preceded by --spin-up seconds (default 0.3) of the same
launch, untimed, then the W warm-up steps: an idle device runs its first milliseconds of work at lower clocks.
Prints ONE JSON line:

  metric/value/unit : weight bytes as stored (packed + fp16 scales, the reference's own definition,
                      scripts/eval/ternary_kernel_bench.py:75-79) per second of wall time over K steps
  roofline          : the same bytes over the kernel's own average duration (HIP events on the
                      launch stream) against the 8 TB/s HBM peak
  cpu_baseline      : the reference's CPU kernel (oracle/_ref, "reference") or this repository's C
                      port of it ("port") timed on the host cores on one linear of the same workload
  also              : secondary measurements (other M, the TQ2 / int8 variants of the GEMV, single-linear
                      latency, grouped-expert GEMM TFLOP/s, prefill / decode tok/s of the decoder harness)
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0
GROUP = 128

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each counter scaled by what it reads for a
# plain 1 GiB device copy) are kept in profiles/hbm_traffic.json, keyed by workload, with the kernel they were
# measured on: the figure is only printed while that kernel is still the one the launch runs.
TRAFFIC_FILE = ROOT / "profiles" / "hbm_traffic.json"


def measured_traffic(workload, kernel):
    try:
        rec = json.loads(TRAFFIC_FILE.read_text()).get(workload)
    except (OSError, ValueError):
        return None
    if not rec or rec.get("kernel") != kernel:
        return None
    return int(rec["fetch_bytes"]) + int(rec["write_bytes"])


def arithmetic_of(kernel):
    """What the kernel named by bp_last_kernel() multiplies in (the `dtype` field of the line is the activation type)."""
    if kernel.startswith("fp4_tq1_t1"):
        return "activations as 3 E4M3 pieces under a per-group power-of-two prescale x E2M1 weights (v_mfma_f32_16x16x128_f8f6f4), fp32 accumulate, fp16 scale per 128-group applied in fp32"
    if kernel.startswith("fp4_tq2"):
        return "activations as 3 E4M3 pieces under a per-group power-of-two prescale (int8 activations: exact) x 2-bit codes read as E2M1 halves with the offset in the accumulator (v_mfma_f32_16x16x128_f8f6f4), fp32 accumulate, fp16 scale per 128-group applied in fp32"
    if kernel.startswith("fp4_tq1_m"):
        return "activations as 2 E4M3 pieces under a per-group power-of-two prescale x E2M1 weights (v_mfma_f32_16x16x128_f8f6f4), fp32 accumulate"
    if kernel.startswith("gemm_tq1f"):
        return "activations as 2 E4M3 pieces under E8M0 block scales (blocks of 32), converted once into a workspace, x E2M1 weights strung together from a byte table, one v_mfma_scale_f32_16x16x128_f8f6f4 per 128-group, fp32 accumulate, scale per group applied in fp32"
    if kernel.startswith("gemm_tq1"):
        return "activations as 2 E4M3 pieces under E8M0 block scales (blocks of 20) x E2M1 weights (v_mfma_scale_f32_16x16x128_f8f6f4), fp32 accumulate, scale per 128-group applied in fp32"
    if kernel.startswith("gemm_tq2f"):
        return "activations as 2 E4M3 pieces under E8M0 block scales (blocks of 32), converted once into a workspace, x E2M1 weights (v_mfma_scale_f32_16x16x128_f8f6f4), fp32 accumulate, scale per 128-group applied in fp32"
    if kernel.startswith(("mfma_tq2_bf16", "gemm_tq2_bf16", "mfma_tq1")):
        return "bf16 activations x bf16-decoded trits (v_mfma_f32_16x16x32_bf16), fp32 accumulate, scale per 128-group applied in fp32"
    if kernel.startswith(("mfma_tq2_i8", "gemm_tq2_i8")):
        return "int8 activations x int8 digits (v_mfma_i32_16x16x64_i8), exact int32 group sums, scales applied in fp32"
    if kernel.startswith("lut_tq1"):
        return "fp32 partial-sum tables, fp32 accumulate"
    return "fp32 (reference operation order)"

SPIN_UP_S = 0.3  # untimed repetitions of a launch before its warm-up and timed steps (see Launch.time)

WORKLOADS = {
    # name: (fmt, N, K, M tokens per linear, activation, terms, L linears per launch)
    "cfg1a_tq1_gemv": ("tq1", 2048, 7168, 1, "bf16", 1, 128),
    "cfg1b_tq1_gemv": ("tq1", 7168, 2048, 1, "bf16", 1, 128),
    "cfg1a_tq1_m2": ("tq1", 2048, 7168, 2, "bf16", 1, 128),
    "cfg1a_tq1_m4": ("tq1", 2048, 7168, 4, "bf16", 1, 128),
    "cfg1a_tq1_m3": ("tq1", 2048, 7168, 3, "bf16", 1, 128),
    "cfg1a_tq1_m6": ("tq1", 2048, 7168, 6, "bf16", 1, 128),
    "cfg1a_tq1_m8": ("tq1", 2048, 7168, 8, "bf16", 1, 128),
    "cfg1a_tq1_m16": ("tq1", 2048, 7168, 16, "bf16", 1, 128),
    "cfg1a_tq1_m32": ("tq1", 2048, 7168, 32, "bf16", 1, 128),
    "cfg1b_tq1_m16": ("tq1", 7168, 2048, 16, "bf16", 1, 128),
    "cfg1b_tq1_m32": ("tq1", 7168, 2048, 32, "bf16", 1, 128),
    "cfg1a_tq2_m2": ("tq2", 2048, 7168, 2, "bf16", 1, 128),
    "cfg1a_tq2_m4": ("tq2", 2048, 7168, 4, "bf16", 1, 128),
    "cfg1a_tq2_m8": ("tq2", 2048, 7168, 8, "bf16", 1, 128),
    "cfg1a_tq2_m16": ("tq2", 2048, 7168, 16, "bf16", 1, 128),
    "cfg1a_tq2_gemv": ("tq2", 2048, 7168, 1, "bf16", 1, 128),
    "cfg0_tq2_gemv": ("tq2", 2048, 4096, 1, "bf16", 1, 192),
    "cfg1a_tq2_i8_gemv": ("tq2", 2048, 7168, 1, "int8", 1, 128),
    "cfg1a_tq1_gemv_L256": ("tq1", 2048, 7168, 1, "bf16", 1, 256),  # twice the linears per launch: the launch's fixed part against twice the bytes
    "cfg1a_tq2_gemv_L256": ("tq2", 2048, 7168, 1, "bf16", 1, 256),
    "cfg1a_tq1_one_linear": ("tq1", 2048, 7168, 1, "bf16", 1, 1),  # what one TernaryLinear call issues (latency-bound: 3 MB)
}


def synth(bp, torch, E, N, K, fmt, terms, seed=0):
    """Draw order (device generator, seed given): per term, per expert: uniform [N, K] -> trits with
    P(-1) = P(+1) = 0.33, P(0) = 0.34; then all scales fp16(0.02 |N(0,1)|) [E, N, G]; later terms reuse
    the first term's scales times 0.25."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    packed, scales = [], []
    for t in range(terms):
        p = torch.empty(E, N, bp.packed_cols(fmt, K), dtype=torch.uint8, device="cuda")
        for e in range(E):
            u = torch.rand(N, K, device="cuda", generator=g)
            p[e] = bp.pack(torch.where(u < 0.33, -1, torch.where(u < 0.66, 1, 0)).to(torch.int8), fmt)
        if t == 0:
            s0 = (0.02 * torch.randn(E, N, K // GROUP, device="cuda", generator=g).abs()).half()
            scales.append(s0)
        else:
            scales.append((s0.float() * 0.25).half())
        packed.append(p)
    return packed, scales


def weight_bytes(packed, scales):
    return sum(p.numel() + 2 * s.numel() for p, s in zip(packed, scales))


class Launch:
    """One grouped launch over E experts with `rows[e]` token rows each, through the native entry."""

    def __init__(self, bp, torch, packed, scales, K, fmt, x, offsets, max_rows, x_scale=None):
        self.e, self.torch = bp.ext(), torch
        self.args = (x, x_scale, offsets, packed, scales, K, GROUP, 2 if fmt == "tq2" else 1, None, max_rows)
        self.out = torch.zeros(x.size(0), packed[0].size(1), dtype=torch.float32, device="cuda")

    def __call__(self):
        self.e.ternary_grouped_gemm(self.out, *self.args)

    def time(self, steps, warmup, spin_up_s=None):
        """`warmup` untimed launches, then `steps` timed ones. Before both, the same launch is repeated for
        `spin_up_s` seconds, untimed: a device that has been idle (a fresh process) runs its first few
        milliseconds of work at lower clocks - 50 launches after 5 warm-up launches measured 114-121 us per launch
        where 200 after the spin-up measure 107-109 us on the same box - and the figure wanted is the steady state."""
        torch = self.torch
        t_end = time.perf_counter() + (SPIN_UP_S if spin_up_s is None else spin_up_s)
        while time.perf_counter() < t_end:
            for _ in range(50):
                self()
            torch.cuda.synchronize()
        for _ in range(warmup):
            self()
        # The boxes show an occasional stall of ~30 ms in the middle of back-to-back launches (about one per several
        # seconds, whatever the kernel). A timed sequence in which one launch took more than 20 x the median launch
        # is taken again, once; `self.retimed` says so and `self.stalled` keeps what the discarded sequence measured
        # (its mean and its slowest launch, in microseconds).
        self.retimed, self.stalled = 0, None
        for attempt in range(2):
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for a, b in ev:
                a.record()
                self()
                b.record()
            torch.cuda.synchronize()
            wall_ev = (time.perf_counter() - t0) / steps
            each = sorted(a.elapsed_time(b) for a, b in ev)
            if attempt == 0 and steps >= 5 and each[-1] > 20.0 * each[len(each) // 2]:
                self.retimed = 1
                self.stalled = {"mean_us": round(sum(each) / steps * 1e3, 2), "slowest_launch_us": round(each[-1] * 1e3, 1),
                                "median_us": round(each[len(each) // 2] * 1e3, 2), "wall_us_per_step": round(wall_ev * 1e6, 2)}
                continue
            break
        kern = sum(each) / steps / 1e3
        # the spread of the per-launch times (HIP events around each launch, microseconds)
        self.spread = {"median": round(each[len(each) // 2] * 1e3, 2), "min": round(each[0] * 1e3, 2), "max": round(each[-1] * 1e3, 2)}
        # The wall-clock figure comes from a sequence of its own, `steps` launches back to back between two
        # synchronisations with nothing else on the stream: the two event records per launch of the sequence above cost
        # about 4.5 us of host time each and keep the next launch from being queued behind the running one.
        for attempt in range(2):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                self()
            torch.cuda.synchronize()
            wall = (time.perf_counter() - t0) / steps
            if attempt == 0 and steps >= 5 and wall * steps > wall_ev * steps + 20.0 * each[len(each) // 2] * 1e-3:  # a stall, as above
                self.retimed = 1
                self.stalled = self.stalled or {"wall_us_per_step": round(wall * 1e6, 2), "median_us": round(each[len(each) // 2] * 1e3, 2)}
                continue
            break
        self.wall_with_events = wall_ev
        return wall, kern, self.e.last_kernel()


def wall_per_call(torch, f, reps, warmup):
    """Seconds per call of f over `reps` back-to-back calls (wall clock around a synchronised sequence); the faster of
    two such sequences, so that one of the boxes' occasional ~30 ms stalls does not end up in the figure."""
    for _ in range(warmup):
        f()
    best = None
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            f()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / reps
        best = dt if best is None or dt < best else best
    return best


def uniform_launch(bp, torch, fmt, N, K, M, act, terms, L, seed=0):
    packed, scales = synth(bp, torch, L, N, K, fmt, terms, seed)
    g = torch.Generator(device="cuda").manual_seed(seed + 1)
    x = torch.randn(L * M, K, device="cuda", generator=g).to(torch.bfloat16)
    xs = None
    if act == "int8":
        x, xs = bp.quant_act_int8(x)
    offsets = torch.arange(0, L * M + 1, M, device="cuda", dtype=torch.int64)
    return Launch(bp, torch, packed, scales, K, fmt, x, offsets, M, xs), weight_bytes(packed, scales)


def cpu_baseline(fmt, N, K, M, budget_s=12.0):
    """Times the CPU ternary kernel on one linear of the workload (float32 activations, as the
    reference's float path takes them) for about `budget_s` seconds of CPU work."""
    import numpy as np

    sys.path.insert(0, str(ROOT / "tests"))
    from _util import c_gemm, orc, oracle_c, ref_gemm, reference_build, synth_trits

    rng = np.random.default_rng(0)
    trits = synth_trits(rng, (N, K))
    scale = (0.02 * np.abs(rng.standard_normal((N, K // GROUP)))).astype(np.float16).astype(np.float32)
    packed = orc.pack(trits, fmt)
    x = rng.standard_normal((M, K)).astype(np.float32)
    kind = "reference" if reference_build() is not None else "port"
    fn = (lambda: ref_gemm(x, None, packed, scale, K, GROUP, fmt)) if kind == "reference" else \
         (lambda: c_gemm(x, None, packed, scale, K, GROUP, fmt))
    for _ in range(3):
        fn()
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s and reps < 20000:
        fn()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    wbytes = packed.size + 2 * scale.size
    cores = oracle_c().bp_oracle_max_threads()
    # the same kernel at 4 threads, the reference's habitual setting (docs/reports/M2.md:114, boilerplate/cli.py:384)
    import torch

    before = torch.get_num_threads()
    torch.set_num_threads(4)  # sets the OpenMP team size the compiled reference kernel uses
    fn4 = fn if kind == "reference" else (lambda: c_gemm(x, None, packed, scale, K, GROUP, fmt, threads=4))
    fn4()
    r4, t1 = 0, time.perf_counter()
    while time.perf_counter() - t1 < budget_s / 3 and r4 < 20000:
        fn4()
        r4 += 1
    dt4 = (time.perf_counter() - t1) / r4
    torch.set_num_threads(before)
    return {"value": round(wbytes / dt / 1e9, 3), "unit": "GB/s", "cores": int(cores), "kind": kind,
            "sample": f"one {fmt} linear N={N} K={K} M={M} fp32 activations, {reps} calls, {dt * 1e3:.3f} ms/call, "
                      f"OpenMP over all {cores} host threads (os.cpu_count()={os.cpu_count()})",
            "value_4_threads": round(wbytes / dt4 / 1e9, 3)}


def skewed_offsets(torch, T, E, k, seed=0):
    """top-k of softmax(N(0, 1.5) logits) per token -> per-expert row counts (skewed loads)."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    logits = torch.randn(T, E, device="cuda", generator=g) * 1.5
    idx = torch.topk(torch.softmax(logits, -1), k, -1).indices.reshape(-1)
    return idx


def cfg3_grouped_launch(bp, torch):
    """The grouped-expert prefill GEMM of config 3: TQ2, two stacked terms, all 384 experts, 2048 tokens top-6 (skewed routing)."""
    from deepseekternarized_amd.kernels.ternary_hip import gather_rows

    E3, N3, K3, T3, k3 = 384, 2048, 4096, 2048, 6
    packed, scales = synth(bp, torch, E3, N3, K3, "tq2", 2, seed=3)
    ids = skewed_offsets(torch, T3, E3, k3, seed=3)
    order, offsets = bp.sort_by_expert(ids, E3)
    xg = gather_rows(torch.randn(T3, K3, device="cuda").to(torch.bfloat16), order, k3)
    max_rows = int((offsets[1:] - offsets[:-1]).max())
    launch = Launch(bp, torch, packed, scales, K3, "tq2", xg, offsets, max_rows)
    flops = 2.0 * T3 * k3 * N3 * K3 * 2  # per-term count
    desc = (f"cfg3 gate projection, E={E3} experts: TQ2 k=2, N={N3}, K={K3}, {T3 * k3} routed rows (max {max_rows}/expert), "
            "bf16 activations")
    return launch, flops, weight_bytes(packed, scales), desc, (packed, scales)


def cfg2_moe(bp, torch):
    """One MoE layer of config 2 (TQ1, H=4096, I=2048, 64 experts, top-6, bf16 activations) as a TernaryMoE."""
    from deepseekternarized_amd.moe import TernaryMoE

    H2, I2, E2, k2 = 4096, 2048, 64, 6
    gate = synth(bp, torch, E2, I2, H2, "tq1", 1, seed=5)
    up = synth(bp, torch, E2, I2, H2, "tq1", 1, seed=6)
    down = synth(bp, torch, E2, H2, I2, "tq1", 1, seed=7)
    layer_bytes = sum(weight_bytes(*m) for m in (gate, up, down))
    moe = TernaryMoE([(gate[0][0], gate[1][0])], [(up[0][0], up[1][0])], [(down[0][0], down[1][0])], H2, I2, k2, "tq1", GROUP, act="bf16")
    return moe, layer_bytes, (H2, I2, E2, k2)


def cfg3_moe(bp, torch, gate=None):
    """One routed-expert layer of config 3 (TQ2, two stacked terms, H=4096, I=2048, 384 experts, top-6, bf16 activations)
    as a TernaryMoE with 2048 tokens of input; `gate`: (packed, scales) of the gate projection if the caller has them."""
    from deepseekternarized_amd.moe import TernaryMoE

    E3, I3, H3, T3, k3 = 384, 2048, 4096, 2048, 6
    packed, scales = gate if gate is not None else synth(bp, torch, E3, I3, H3, "tq2", 2, seed=3)
    up3 = synth(bp, torch, E3, I3, H3, "tq2", 2, seed=4)
    down3 = synth(bp, torch, E3, H3, I3, "tq2", 2, seed=5)
    moe3 = TernaryMoE(list(zip(packed, scales)), list(zip(*up3)), list(zip(*down3)), H3, I3, k3, "tq2", GROUP, act="bf16")
    g3 = torch.Generator(device="cuda").manual_seed(9)
    x3 = torch.randn(T3, H3, device="cuda", generator=g3).to(torch.bfloat16)
    lg3 = torch.randn(T3, E3, device="cuda", generator=g3) * 1.5
    fl3 = 2.0 * T3 * k3 * 3 * H3 * I3 * 2  # per-term count, three projections
    desc = (f"TQ2 k=2 MoE layer H={H3} I={I3} E={E3} top-{k3}, {T3} tokens, bf16 activations: softmax/top-k, "
            "sort, gate|up grouped GEMM (row gather in its conversion pass, SwiGLU in its epilogue), down grouped GEMM, weighted combine")
    return moe3, x3, lg3, fl3, desc


def run_cfg3_moe(bp, torch, a) -> int:
    moe3, x3, lg3, fl3, desc = cfg3_moe(bp, torch)
    t_end = time.perf_counter() + SPIN_UP_S
    while time.perf_counter() < t_end:
        moe3(x3, lg3)
        torch.cuda.synchronize()
    dt = wall_per_call(torch, lambda: moe3(x3, lg3), a.steps, a.warmup)
    kname = bp.ext().last_kernel()
    return emit({
        "metric": "ternary GEMV HBM GB/s (% peak); grouped-expert GEMM TFLOP/s (% MFMA peak)",
        "value": round(fl3 / dt / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3_moe: " + desc, "kernel": kname, "arithmetic": arithmetic_of(kname.split("+")[0]),
                   "flops_counted": "2 x routed rows x N x K per term (two terms), three projections", "device_spin_up_s": SPIN_UP_S},
        "roofline": {"bound": "mfma", "achieved": round(fl3 / dt / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(fl3 / dt / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None, "layer_us": round(dt * 1e6, 2),
                     "note": "whole layer (seven launches) by wall clock, not one kernel"},
        "cpu_baseline": None, "also": {}})


def huffman_stream(torch, n, seed=0, repeat=1):
    """A Mode B stream of n symbols made here with numpy (the package has the decoder only): a skewed byte distribution
    under a canonical code of lengths 2 / 4 / 6 / 8 / 12, MSB first, codes back to back, a bit offset per block of 4096
    symbols (boilerplate/kernels/csrc/boilerplate_cpu.cpp:133-167)."""
    import numpy as np

    from deepseekternarized_amd import entropy

    lens = np.full(256, 12, np.uint8)
    lens[:2], lens[2:6], lens[6:14], lens[14:30] = 2, 4, 6, 8
    codes = entropy.canonical_codes(torch.from_numpy(lens)).numpy().astype(np.int64)
    p = 2.0 ** -lens.astype(np.float64)
    rng = np.random.default_rng(seed)
    sym = rng.choice(256, size=n, p=p / p.sum()).astype(np.uint8)
    L = lens[sym].astype(np.int64)
    if repeat > 1:  # whole bytes and whole blocks, so that the stream can be laid end to end: a few 2-bit codes become 4-bit ones
        assert n % entropy.BLOCK == 0
        short = np.flatnonzero(L == 2)[-3:]
        fix = short[: ((8 - int(L.sum()) % 8) % 8) // 2]
        sym[fix] = 2
        L[fix] = 4
    block = entropy.BLOCK
    nb = -(-n // block)
    starts = np.concatenate([[0], np.cumsum(L)]).astype(np.int64)  # first bit of every symbol's code: codes back to back
    offsets = np.concatenate([starts[:-1][::block][:nb], [starts[-1]]]).astype(np.int64)  # bit where a block starts; last: the total
    bits = np.zeros(int(starts[-1]), np.uint8)
    c = codes[sym]
    for j in range(12):
        m = L > j
        bits[starts[:-1][m] + j] = (c[m] >> (L[m] - 1 - j)) & 1
    packed = np.packbits(bits)
    if repeat > 1:
        offsets = np.concatenate([offsets[:-1] + r * int(starts[-1]) for r in range(repeat)] + [[repeat * int(starts[-1])]]).astype(np.int64)
        packed, sym = np.tile(packed, repeat), np.tile(sym, repeat)
    stream = np.zeros(packed.size + 8, np.uint8)  # (zero padding behind the last code, as the reference's encoder leaves it)
    stream[: packed.size] = packed
    return {"stream": torch.from_numpy(stream).cuda(), "offsets": torch.from_numpy(offsets), "lens": torch.from_numpy(lens)}, sym


def huff_case(bp, torch, entropy, timed, res, n_sym, repeat, name):
    parts, sym = huffman_stream(torch, n_sym // repeat, repeat=repeat)
    sym_d = torch.from_numpy(sym).cuda()
    buf = torch.empty(n_sym, dtype=torch.uint8, device="cuda")
    assert torch.equal(entropy.decode(parts, n_sym, out=buf), sym_d)
    # (timed through the C entry point with the tables made once: the Python wrapper builds the decode table on the host
    # and reads the error flag back, about a millisecond per call)
    from deepseekternarized_amd.kernels import _lib
    lut_host = entropy.decode_table(parts["lens"], entropy.MAXLEN)
    lut, off_d, flag = lut_host.cuda(), parts["offsets"].cuda(), torch.zeros(1, dtype=torch.int32, device="cuda")
    lib = bp.ext().lib

    def huff():
        _lib.check(lib.bp_huff_decode(buf.data_ptr(), buf.numel(), parts["stream"].data_ptr(), parts["stream"].numel(), off_d.data_ptr(),
                                      parts["offsets"].data_ptr(), n_sym, entropy.BLOCK, lut.data_ptr(), lut_host.data_ptr(), entropy.MAXLEN,
                                      None, 0, flag.data_ptr(), _lib.stream_ptr(buf.device)))
        return buf

    timed(name, huff, parts["stream"].numel() + n_sym, check=lambda o: torch.equal(o, sym_d) and int(flag.item()) == 0)
    res[name]["bits_per_symbol"] = round(8 * parts["stream"].numel() / n_sym, 2)
    del parts, sym_d, buf, lut, off_d


def aux_kernels(bp, torch, steps, big=True):
    """The kernels either side of the GEMMs - pack / unpack, the scale and activation conversions, the absmean producer,
    GGUF blocks, Mode B's decode, routing - each timed alone on a tensor of config 1's size (16 linears of 2048 x 7168),
    bytes counted as what the operation has to read and write once."""
    import numpy as np

    from deepseekternarized_amd import entropy, gguf_blocks
    from deepseekternarized_amd.kernels.ternary_hip import gather_rows
    from deepseekternarized_amd.ternary import fit
    from deepseekternarized_amd.ternary.ops import PackedTerm
    from deepseekternarized_amd.ternary.pack import expand_scales

    N, K = 16 * 2048, 7168
    g = torch.Generator(device="cuda").manual_seed(1)
    w = torch.randn(N, K, device="cuda", generator=g) * 0.02
    trits = torch.randint(-1, 2, (N, K), device="cuda", generator=g, dtype=torch.int8)
    res = {}

    def timed(name, f, nbytes, check=None):
        out = f()
        torch.cuda.synchronize()
        if check is not None:
            assert check(out), name
        reps = max(5, min(steps, 30))
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for e0, e1 in ev:
            e0.record()
            f()
            e1.record()
        torch.cuda.synchronize()
        t = sorted(e0.elapsed_time(e1) for e0, e1 in ev)[reps // 2] * 1e-3
        res[name] = {"us": round(t * 1e6, 1), "GBps": round(nbytes / t / 1e9, 1), "frac_of_hbm_peak": round(nbytes / t / 1e9 / HBM_PEAK_GBPS, 4),
                     "bytes": int(nbytes)}
        return out

    for fmt in ("tq1", "tq2"):
        kp = bp.packed_cols(fmt, K)
        pk = timed(f"pack_{fmt}", lambda: bp.pack(trits, fmt), N * K + N * kp)
        timed(f"unpack_{fmt}", lambda: bp.unpack(pk, fmt, K), N * kp + N * K, check=lambda o: torch.equal(o, trits))
        timed(f"absmean_pack_{fmt}_f32", lambda: fit.packed_term(w, 128, fmt), 4 * N * K + N * kp + 2 * N * K // 128)
    wb = w.to(torch.bfloat16)
    timed("absmean_pack_tq2_bf16", lambda: fit.packed_term(wb, 128, "tq2"), 2 * N * K + N * K // 4 + 2 * N * K // 128)
    sc = (torch.rand(N, K // 128, device="cuda", generator=g) + 0.5).half()
    timed("expand_scales_f16", lambda: expand_scales(sc), 6 * sc.numel())
    x = torch.randn(4096, K, device="cuda", generator=g).to(torch.bfloat16)
    timed("quant_act_int8_bf16", lambda: bp.quant_act_int8(x), x.numel() * 3 + 4 * x.size(0))
    # GGUF blocks: single-term, group-256, fp16 scales
    sc256 = (torch.rand(N, K // 256, device="cuda", generator=g) + 0.5).half()
    for fmt, q in (("tq1", "tq1"), ("tq2", "tq2")):
        kp = bp.packed_cols(fmt, K)
        term = PackedTerm(bp.pack(trits, fmt), sc256)
        bs = 54 if q == "tq1" else 66
        blocks = timed(f"gguf_{q}_0_from_{fmt}", lambda: gguf_blocks.to_gguf_blocks(term, K, fmt, 256, q), N * kp + 2 * sc256.numel() + N * K // 256 * bs)
        timed(f"gguf_{q}_0_to_{fmt}", lambda: gguf_blocks.from_gguf_blocks(blocks, K, fmt, q), N * K // 256 * bs + N * kp + 2 * sc256.numel(),
              check=lambda o: torch.equal(o.packed, term.packed) and torch.equal(o.scale, sc256))
        del term, blocks
    # Mode B decode, one-byte format: 64 Mi symbols (16,384 blocks: one lane each, one wave per CU) and 1 Gi symbols
    for n_sym, rep_, name in ((64 << 20, 1, "huff_decode_u8_64Mi"), (1 << 30, 16, "huff_decode_u8_1Gi"))[: 2 if big else 1]:
        huff_case(bp, torch, entropy, timed, res, n_sym, rep_, name)
    # routing: config 3's 12,288 ids over 384 experts, and a million ids
    for n_ids, E in ((12288, 384), (1 << 20, 384)):
        ids = torch.randint(0, E, (n_ids,), device="cuda", generator=g)
        timed(f"sort_by_expert_{n_ids}", lambda: bp.sort_by_expert(ids, E), 8 * n_ids * 2 + 8 * E)
    xs = torch.randn(2048, 4096, device="cuda", generator=g).to(torch.bfloat16)
    order, _ = bp.sort_by_expert(torch.randint(0, 384, (12288,), device="cuda", generator=g), 384)
    timed("gather_rows_12288x4096_bf16", lambda: gather_rows(xs, order, 6), 2 * 12288 * 4096 * 2)
    return res, (N, K)


def aux_cpu_baseline(K, rows=512):
    """The NumPy restatements of the same operations on `rows` rows of the same width, one host thread: bytes read +
    written once per second, for the figure beside the device's."""
    import numpy as np

    sys.path.insert(0, str(ROOT / "tests"))
    from _util import orc

    rng = np.random.default_rng(0)
    trits = rng.integers(-1, 2, (rows, K)).astype(np.int8)
    w = (rng.standard_normal((rows, K)) * 0.02).astype(np.float32)
    out = {}

    def timed(name, f, nbytes):
        f()
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 1.0:
            f()
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        out[name] = {"GBps": round(nbytes / dt / 1e9, 3), "ms": round(dt * 1e3, 2)}

    for fmt in ("tq1", "tq2"):
        kp = orc.packed_cols(fmt, K)
        pk = orc.pack(trits, fmt)
        timed(f"pack_{fmt}", lambda: orc.pack(trits, fmt), rows * (K + kp))
        timed(f"unpack_{fmt}", lambda: orc.unpack(pk, fmt, K), rows * (K + kp))
    timed("absmean_ternary_f32", lambda: orc.absmean_ternary(w, 128, "f16"), rows * (4 * K + K + 2 * K // 128))
    x = orc.bf16_round(rng.standard_normal((rows, K)).astype(np.float32))
    timed("quant_act_int8", lambda: orc.quant_act_int8(x), rows * (3 * K + 4))
    return {"value": out["pack_tq1"]["GBps"], "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"NumPy restatements on {rows} x {K}, about a second each, one host thread", "each": out}


def run_aux_kernels(bp, torch, a) -> int:
    res, (N, K) = aux_kernels(bp, torch, a.steps)
    cpu = None if a.no_cpu else aux_cpu_baseline(K)
    worst = min(res, key=lambda k: res[k]["frac_of_hbm_peak"] if res[k]["bytes"] > (64 << 20) else 9.0)
    return emit({
        "metric": "ternary GEMV HBM GB/s (% peak); grouped-expert GEMM TFLOP/s (% MFMA peak)",
        "value": res[worst]["GBps"], "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(res[worst]["us"] * 1e-3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"aux_kernels: producer, format and routing kernels alone on {N} x {K} weights (value: the slowest large one, {worst})",
                   "bytes_counted": "inputs read once + outputs written once; median of the timed calls by HIP events, Python wrapper and output allocation included"},
        "roofline": {"bound": "hbm", "achieved": res[worst]["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": res[worst]["frac_of_hbm_peak"],
                     "traffic": None, "kernel": worst},
        "cpu_baseline": cpu, "also": res})


def emit(line) -> int:
    print(json.dumps(line))
    return 0


def run_cfg3_grouped(bp, torch, a) -> int:
    launch, flops, wbytes, desc, _ = cfg3_grouped_launch(bp, torch)
    wall, kern, kname = launch.time(a.steps, a.warmup)
    return emit({
        "metric": "ternary GEMV HBM GB/s (% peak); grouped-expert GEMM TFLOP/s (% MFMA peak)",
        "value": round(flops / wall / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "cfg3_grouped: " + desc, "kernel": kname, "arithmetic": arithmetic_of(kname),
                   "flops_counted": "2 x routed rows x N x K per term (two terms)", "device_spin_up_s": SPIN_UP_S,
                   "retimed_after_stall": launch.retimed, "weight_GBps": round(wbytes / kern / 1e9, 1)},
        "roofline": {"bound": "mfma", "achieved": round(flops / kern / 1e12, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops / kern / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": measured_traffic("cfg3_grouped", kname),
                     "kernel_us": round(kern * 1e6, 2), "kernel_us_median": launch.spread["median"], "kernel_us_min": launch.spread["min"],
                     "kernel_us_max": launch.spread["max"]},
        "cpu_baseline": None, "also": {}})


def run_cfg2_moe(bp, torch, a, T2) -> int:
    moe, layer_bytes, (H2, I2, E2, k2) = cfg2_moe(bp, torch)
    gm = torch.Generator(device="cuda").manual_seed(8)
    xt = torch.randn(T2, H2, device="cuda", generator=gm).to(torch.bfloat16)
    lg = torch.randn(T2, E2, device="cuda", generator=gm) * 1.5
    t_end = time.perf_counter() + SPIN_UP_S
    while time.perf_counter() < t_end:
        moe(xt, lg)
        torch.cuda.synchronize()
    dt = wall_per_call(torch, lambda: moe(xt, lg), a.steps, a.warmup)
    active = int(torch.unique(torch.topk(torch.softmax(lg.float(), -1), k2, -1).indices).numel())
    kname = bp.ext().last_kernel()
    abytes = layer_bytes / E2 * active
    return emit({
        "metric": "ternary GEMV HBM GB/s (% peak); grouped-expert GEMM TFLOP/s (% MFMA peak)",
        "value": round(abytes / dt / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(dt * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"cfg2_moe_T{T2}: TQ1 MoE layer H={H2} I={I2} E={E2} top-{k2}, {T2} tokens, bf16 activations: softmax/top-k, sort, "
                               f"gather, gate|up grouped GEMM, SwiGLU, down grouped GEMM, weighted combine (beyond 24 tokens the gate|up launch gathers its rows and applies SwiGLU itself); {active} active experts",
                   "kernel": kname, "arithmetic": arithmetic_of(kname), "bytes_counted": "packed + fp16 scales of the active experts",
                   "device_spin_up_s": SPIN_UP_S},
        "roofline": {"bound": "hbm", "achieved": round(abytes / dt / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(abytes / dt / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None, "layer_us": round(dt * 1e6, 2),
                     "note": "whole layer (a dozen launches) by wall clock, not one kernel"},
        "cpu_baseline": None, "also": {}})


def run_cfg4_decoder(bp, torch, a, graph: bool) -> int:
    """Config 4: the OLMoE-shaped Mode D decoder harness, batch 64, 128 prompt + 128 greedy decode tokens (one HIP graph
    per decode step with `graph`); value = decode tokens per second."""
    from deepseekternarized_amd.decoder_harness import DecoderConfig, TernaryDecoder, bench_decoder

    cfg = DecoderConfig()
    model = TernaryDecoder(cfg)
    r = bench_decoder(model, 64, 128, 128, graph=graph)
    weight_bytes_per_step = cfg.layers * (4 * (cfg.hidden * cfg.hidden // 4 + 2 * cfg.hidden * cfg.hidden // GROUP)
                                          + cfg.experts * 3 * (cfg.inter * cfg.hidden // 4 + 2 * cfg.inter * cfg.hidden // GROUP))
    step_s = 64.0 / r["decode_tok_s"]
    return emit({
        "metric": "ternary GEMV HBM GB/s (% peak); grouped-expert GEMM TFLOP/s (% MFMA peak)",
        "value": round(r["decode_tok_s"], 1), "unit": "tok/s", "n_gpus": 1, "steps": 128, "warmup": 0,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg.act, "data": "synthetic",
        "config": {"workload": f"cfg4_decode{'_graph' if graph else ''}: {cfg.layers} layers, hidden {cfg.hidden}, {cfg.experts} experts top-{cfg.top_k}, inter {cfg.inter}, "
                               f"{cfg.fmt.upper()}, {cfg.act} activations, random weights; batch 64, prompt 128, 128 greedy decode steps",
                   "prefill_tok_s": r["prefill_tok_s"], "peak_vram_bytes": r["peak_vram_bytes"], "finite": r["finite"]},
        "roofline": {"bound": "hbm", "achieved": round(weight_bytes_per_step / step_s / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(weight_bytes_per_step / step_s / 1e9 / HBM_PEAK_GBPS, 4), "traffic": None,
                     "note": "all ternary weights of the model (every expert is active at batch 64) per decode step by wall clock; not one kernel"},
        "cpu_baseline": None, "also": {}})


def main() -> int:
    global SPIN_UP_S
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spin-up", type=float, default=SPIN_UP_S, help="seconds of untimed launches before warm-up and timed steps (0: none, for counter runs)")
    ap.add_argument("--workload", default="cfg1a_tq1_gemv", choices=sorted(WORKLOADS) + ["aux_kernels", "cfg3_grouped", "cfg3_moe", "cfg2_moe_T1", "cfg2_moe_T32", "cfg2_moe_T256", "cfg4_decode", "cfg4_decode_graph"])
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="instead of the workload, run a plain 1 GiB device-to-device copy `steps` times "
                         "(the known-size kernel that FETCH_SIZE / WRITE_SIZE counter readings are scaled by)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch

    import deepseekternarized_amd as bp

    if not torch.cuda.is_available() or bp.ext() is None:
        print("bench.py needs a HIP device and the built libbp_ternary_hip.so", file=sys.stderr)
        return 1
    if a.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(a.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "device copy", "bytes_read": 1 << 30, "bytes_written": 1 << 30, "steps": a.steps}))
        return 0
    SPIN_UP_S = max(0.0, a.spin_up)
    if a.workload == "cfg3_grouped":
        return run_cfg3_grouped(bp, torch, a)
    if a.workload == "cfg3_moe":
        return run_cfg3_moe(bp, torch, a)
    if a.workload == "aux_kernels":
        return run_aux_kernels(bp, torch, a)
    if a.workload.startswith("cfg2_moe_T"):
        return run_cfg2_moe(bp, torch, a, int(a.workload[len("cfg2_moe_T"):]))
    if a.workload.startswith("cfg4_decode"):
        return run_cfg4_decoder(bp, torch, a, a.workload.endswith("_graph"))
    fmt, N, K, M, act, terms, L = WORKLOADS[a.workload]
    launch, wbytes = uniform_launch(bp, torch, fmt, N, K, M, act, terms, L)
    wall, kern, kname = launch.time(a.steps, a.warmup)
    retimed, stalled, spread = launch.retimed, launch.stalled, launch.spread
    act_bytes = L * M * K * 2 + L * M * N * 4 * 2  # bf16 activations read, f32 output read-modify-write

    also = {}
    if not a.no_extras:
        del launch
        torch.cuda.empty_cache()
        for m in (2, 4, 16, 32):  # the other decode batch sizes of the configuration
            l2, wb2 = uniform_launch(bp, torch, fmt, N, K, m, act, terms, L)
            _, k2, kn2 = l2.time(max(30, a.steps // 2), 5)
            also[f"M{m}_weight_GBps"] = round(wb2 / k2 / 1e9, 1)
            also[f"M{m}_kernel"] = kn2
            also[f"M{m}_us"] = round(k2 * 1e6, 1)
            also[f"M{m}_us_median"] = l2.spread["median"]
            del l2
            torch.cuda.empty_cache()
        for name in ("cfg1a_tq2_gemv", "cfg1a_tq2_i8_gemv", "cfg1b_tq1_gemv"):  # the same GEMV in the other formats / shapes
            if name == a.workload:
                continue
            f2, n2, k2_, m2, act2, t2, L2 = WORKLOADS[name]
            l2, wb2 = uniform_launch(bp, torch, f2, n2, k2_, m2, act2, t2, L2)
            _, kk, kn2 = l2.time(max(30, a.steps // 2), 5)
            also[name] = {"weight_GBps": round(wb2 / kk / 1e9, 1), "frac_of_hbm_peak": round(wb2 / kk / 1e9 / HBM_PEAK_GBPS, 4),
                          "kernel": kn2, "us": round(kk * 1e6, 1), "us_median": l2.spread["median"]}
            del l2
            torch.cuda.empty_cache()
        l1, wb1 = uniform_launch(bp, torch, fmt, N, K, M, act, terms, 1)  # one linear per launch (cache-resident, latency bound)
        w1, k1, _ = l1.time(200, 20)
        also["single_linear_us_per_call"] = round(w1 * 1e6, 2)
        also["single_linear_weight_GBps"] = round(wb1 / w1 / 1e9, 1)
        del l1
        # one MoE layer of config 2 (TQ1, H=4096, I=2048, 64 experts, top-6, bf16 activations) through TernaryMoE
        moe, layer_bytes, (H2, I2, E2, k2) = cfg2_moe(bp, torch)
        gm = torch.Generator(device="cuda").manual_seed(8)
        cfg2 = {}
        for T2 in (1, 32, 256):
            xt = torch.randn(T2, H2, device="cuda", generator=gm).to(torch.bfloat16)
            lg = torch.randn(T2, E2, device="cuda", generator=gm) * 1.5
            reps = 20
            dt = wall_per_call(torch, lambda: moe(xt, lg), reps, 3)
            active = int(torch.unique(torch.topk(torch.softmax(lg.float(), -1), k2, -1).indices).numel())
            cfg2[f"T{T2}"] = {"ms_per_layer": round(dt * 1e3, 4), "active_experts": active,
                              "active_weight_GBps": round(layer_bytes / E2 * active / dt / 1e9, 1)}
            if T2 <= 64:  # the same layer replayed as one HIP graph (launch-bound at a few tokens)
                run = moe.graphed(T2)
                dg = wall_per_call(torch, lambda: run(xt, lg), reps, 3)
                cfg2[f"T{T2}"]["ms_per_layer_hip_graph"] = round(dg * 1e3, 4)
                cfg2[f"T{T2}"]["active_weight_GBps_hip_graph"] = round(layer_bytes / E2 * active / dg / 1e9, 1)
                del run
        also["cfg2_moe_layer"] = {"workload": f"TQ1 MoE layer H={H2} I={I2} E={E2} top-{k2}, bf16 activations: softmax/top-k, sort, gather, "
                                              "gate|up grouped GEMM, SwiGLU, down grouped GEMM, weighted combine", **cfg2}
        del moe
        torch.cuda.empty_cache()
        # grouped-expert prefill GEMM of config 3: TQ2, two stacked terms, all 384 experts, 2048 tokens top-6 (skewed routing)
        E3, N3, K3, T3, k3 = 384, 2048, 4096, 2048, 6
        l3, flops, wb3, desc3, (packed, scales) = cfg3_grouped_launch(bp, torch)
        _, k3t, kn3 = l3.time(max(30, a.steps // 2), 5)
        also["grouped_gemm"] = {"workload": desc3, "TFLOPs_per_term_count": round(flops / k3t / 1e12, 1),
                                "frac_of_bf16_mfma_peak": round(flops / k3t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4),
                                "weight_GBps": round(wb3 / k3t / 1e9, 1), "kernel": kn3, "us": round(k3t * 1e6, 1), "us_median": l3.spread["median"]}
        del l3
        # ... and the whole routed-expert layer of config 3 (gate | up, SwiGLU, down, combine) on the same gate stack
        moe3, x3, lg3, fl3, desc3m = cfg3_moe(bp, torch, gate=(packed, scales))
        del packed, scales
        dt3 = wall_per_call(torch, lambda: moe3(x3, lg3), 10, 3)
        also["cfg3_moe_layer"] = {"workload": desc3m, "kernel": bp.ext().last_kernel(),
                                  "ms_per_layer": round(dt3 * 1e3, 3), "TFLOPs_per_term_count": round(fl3 / dt3 / 1e12, 1),
                                  "frac_of_bf16_mfma_peak": round(fl3 / dt3 / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del moe3, x3, lg3
        torch.cuda.empty_cache()
        # the producer, format and routing kernels either side of the GEMMs, each alone (us, bytes read + written once per second)
        aux, _ = aux_kernels(bp, torch, 10, big=False)
        also["aux_kernels"] = {k: {"us": v["us"], "GBps": v["GBps"]} for k, v in aux.items()}
        torch.cuda.empty_cache()
        # end-to-end timing loop of the reference's `boilerplate bench` on a random-init OLMoE-shaped Mode D decoder
        from deepseekternarized_amd.decoder_harness import DecoderConfig, TernaryDecoder, bench_decoder

        cfg = DecoderConfig()
        model = TernaryDecoder(cfg)
        r = bench_decoder(model, 64, 128, 128)
        rg = bench_decoder(model, 64, 128, 128, graph=True)  # the same decode steps replayed as one HIP graph each
        also["decoder_harness"] = {"workload": f"{cfg.layers} layers, hidden {cfg.hidden}, {cfg.experts} experts top-{cfg.top_k}, "
                                               f"inter {cfg.inter}, {cfg.fmt.upper()}, {cfg.act} activations, random weights; "
                                               "batch 64, prompt 128, 128 greedy decode steps",
                                   "prefill_tok_s": r["prefill_tok_s"], "decode_tok_s": r["decode_tok_s"],
                                   "decode_tok_s_hip_graph": rg["decode_tok_s"],
                                   "peak_vram_bytes": r["peak_vram_bytes"], "finite": r["finite"] and rg["finite"]}

    line = {
        "metric": "ternary GEMV HBM GB/s (% peak); grouped-expert GEMM TFLOP/s (% MFMA peak)",
        "value": round(wbytes / wall / 1e9, 1), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall * 1e3, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{a.workload}: {fmt.upper()} decode GEMV N={N} K={K} M={M} {act} activations, group 128, "
                               f"fp16 scales, {L} distinct linears per launch ({wbytes / 1e6:.0f} MB of weights, > Infinity Cache)",
                   "kernel": kname, "arithmetic": arithmetic_of(kname), "bytes_counted": "packed + fp16 scales as stored", "device_spin_up_s": SPIN_UP_S, "retimed_after_stall": retimed,
                   "discarded_sequence_with_stall": stalled,
                   "packed_only_GBps": round(wbytes * (1.0 - 2.0 * (K // GROUP) / (bp.packed_cols(fmt, K) + 2.0 * (K // GROUP))) / kern / 1e9, 1),
                   "activation_and_output_bytes_per_step": act_bytes},
        "roofline": {"bound": "hbm", "achieved": round(wbytes / kern / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(wbytes / kern / 1e9 / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(a.workload, kname),
                     "kernel_us": round(kern * 1e6, 2), "kernel_us_median": spread["median"], "kernel_us_min": spread["min"],
                     "kernel_us_max": spread["max"],
                     "note": "achieved / frac use the MEAN launch duration over the timed steps (HIP events on the launch stream)"},
        "cpu_baseline": None if a.no_cpu else cpu_baseline(fmt, N, K, M),
        "also": also,
    }
    return emit(line)


if __name__ == "__main__":
    raise SystemExit(main())

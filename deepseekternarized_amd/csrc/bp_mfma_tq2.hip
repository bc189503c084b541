// TQ2 (4 trits per byte) on MFMA: table-free decode, activations and scales staged through LDS.
#include "bp_mfma.h"
#include "bp_tq2_decode.h"

namespace bp {
namespace {

// The activation tile starts at LDS address 0: row t at t * pitch, pitch = KC * XB + 16.
constexpr int X_BASE = 0;
// LDS budget for a workgroup's scales (beyond it: read from global memory)
constexpr int tq2_scale_tile_max(int) { return 40 * 1024; }

// ------------------------------------------------------------------------------------------------
// TQ2. K % 256 == 0, N % 16 == 0. One step = 64 packed bytes (256 trits, two groups) per row.
// Lane (r16 = lane % 16, b = lane / 16) loads bytes [16b, 16b + 16) of its row's 64-byte piece; a
// v_permlane32_swap pair then leaves every lane with 8 bytes of the first group and 8 bytes of the
// second, so that all four k-blocks of an MFMA belong to one scale group.
// After the swap block b holds trits tb(b) .. tb(b)+31 of each group, tb = {0, 64, 32, 96}.
template <int ACT, int SDT, int R, int MT, int WAVES, int XKB, int ABL = 0, int NQ = 4, int SL = 1>
__global__ __launch_bounds__(WAVES * 64, 4) void k_mfma_tq2(GemmArgs a, int KC, int tile_rows) {
  constexpr int THREADS = WAVES * 64;
  constexpr int XB = ACT == BP_BF16 ? 2 : 1;   // bytes per activation element
  constexpr int KM = ACT == BP_BF16 ? 8 : 16;  // k per lane per MFMA
  constexpr int NJ = 32 / KM;                  // MFMAs per group
  constexpr int XU = (XKB * 1024 / (16 * XB) + THREADS - 1) / THREADS;  // 16-element units of the activation tile per thread (rounded up: 16 waves and 16-bit activations hold 1.5 each)
  static_assert(XU * THREADS * 16 * XB >= XKB * 1024, "every unit of the activation tile has a thread that stages it");

  // the wave index through readfirstlane: everything derived from it stays in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, b = lane >> 4;
  const int64_t e = blockIdx.y;
  const int64_t o0 = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  const int64_t tok0 = o0 + (int64_t)blockIdx.z * (16 * MT);
  if (tok0 >= o1) return;  // uniform for the workgroup: no barrier is skipped by part of it
  const int ntok = (int)(o1 - tok0 < 16 * MT ? o1 - tok0 : 16 * MT);
  int64_t n0 = ((int64_t)blockIdx.x * WAVES + wave) * (16 * R);
  const bool wave_live = n0 < a.N;
  if (!wave_live) n0 = 0;  // keeps addresses valid; the wave still takes part in staging and barriers
  const int tb = 64 * (b & 1) + 32 * (b >> 1);

  // row sub-tiles past N re-read the first sub-tile (branch-free loop body) and are dropped at the store
  bool rows_valid[R];
  int64_t row_shift[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    rows_valid[r] = wave_live && n0 + 16 * r < a.N;
    row_shift[r] = rows_valid[r] ? 16 * r : 0;
  }

  // ---- activation tile geometry
  const int pitch = KC * XB + 16;
  const int units_per_row = KC / 16;
  const int units = ntok * units_per_row;
  unsigned xaddr[MT];  // LDS address of this lane's token row (+ its k-block offset)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    int t = 16 * mt + r16;
    if (t >= ntok) t = ntok - 1;
    xaddr[mt] = (unsigned)(X_BASE + t * pitch + tb * XB);
  }
  // Offset removal: corr[g][t] = -sum over the 128 k of group g of x[t, k] * (c(k) + 1) (bf16: c + 1 = 9 for
  // even k, 3 for odd k; int8: 1), float32 / int32, at corr_base + (g * 16 * MT + t) * 4. A lane starts the
  // accumulator of a group from the four values of its tokens 4b .. 4b + 3.
  const unsigned corr_base = (unsigned)(X_BASE + tile_rows * pitch);
  const unsigned corr_lane = corr_base + (unsigned)(16 * b);
  const unsigned char* xg = (const unsigned char*)a.x + tok0 * a.K * XB;
  u32x4 xstage[XU][XB];
  auto stage_load = [&](int64_t k0) {  // global -> registers, chunk starting at k0
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      const int u = threadIdx.x + i * THREADS;
      const int row = u / units_per_row, col = u - row * units_per_row;
      if (u < units && k0 + col * 16 < a.K) {  // the last chunk may be shorter than KC: stay inside the row
        const unsigned char* p = xg + ((int64_t)row * a.K + k0 + col * 16) * XB;
#pragma unroll
        for (int v = 0; v < XB; ++v) xstage[i][v] = *(const u32x4*)(p + 16 * v);
      }
    }
  };
  auto stage_store = [&]() {  // registers -> LDS, every 16 elements reordered to the decode's slot order
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      const int u = threadIdx.x + i * THREADS;
      if (u < units) {
        const int row = u / units_per_row, col = u - row * units_per_row;
        const unsigned dst = (unsigned)(X_BASE + row * pitch + col * 16 * XB);
        unsigned part;  // this unit's share of the group's offset sum; 8 consecutive lanes hold one group
        if (ACT == BP_BF16) {
          u32x4 o0, o1;
          tq2_permute_bf16(xstage[i][0], xstage[i][XB - 1], o0, o1);
          *(lds_u32x4*)(dst) = o0;
          *(lds_u32x4*)(dst + 16) = o1;
          float f = 0.f;
          const bf16x2 w93 = __builtin_bit_cast(bf16x2, 0x40404110u);  // (9.0, 3.0): even k in the low half
#pragma unroll
          for (int v = 0; v < XB; ++v) {
            const unsigned dw[4] = {xstage[i][v].x, xstage[i][v].y, xstage[i][v].z, xstage[i][v].w};
#pragma unroll
            for (int d = 0; d < 4; ++d) f = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, dw[d]), w93, f, false);
          }
          f += __shfl_xor(f, 1);
          f += __shfl_xor(f, 2);
          f += __shfl_xor(f, 4);
          part = __float_as_uint(-f);
        } else {
          *(lds_u32x4*)(dst) = tq2_permute_i8(xstage[i][0]);
          int n = 0;
#pragma unroll
          for (int d = 0; d < 4; ++d) n = __builtin_amdgcn_sdot4((int)xstage[i][0][d], 0x01010101, n, false);
          n += __shfl_xor(n, 1);
          n += __shfl_xor(n, 2);
          n += __shfl_xor(n, 4);
          part = (unsigned)(-n);
        }
        if ((col & 7) == 0) *(lds_u32*)(corr_base + ((col >> 3) * (16 * MT) + row) * 4) = part;
      }
    }
  };

  f32x4 total[R][MT];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) total[r][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // decode masks and exponent patterns live in registers: v_and_or_b32 takes no literal operands
  Tq2Consts kc = {0x00c000c0u, 0x00300030u, 0x40004000u, 0x41004100u};
  asm volatile("" : "+s"(kc.P1), "+s"(kc.P2));
  asm volatile("" : "+v"(kc.M1), "+v"(kc.M2));

  const int steps = (int)(a.K / 256);
  const int gs = a.group == 256 ? 1 : 0;  // scale groups of 256: the two 128-wide halves of a step share a scale (read from global memory)
  const int steps_per_chunk = KC / 256;
  const int chunks = (steps + steps_per_chunk - 1) / steps_per_chunk;

  for (int term = 0; term < a.n_terms; ++term) {
    // this wave's rows of the term as two buffers (R sub-tiles of 16 rows; rows past N are not in range)
    constexpr int SB = SDT == BP_F32 ? 4 : 2;
    const int64_t rows_here = a.N - n0 < 16 * R ? a.N - n0 : 16 * R;
    const __amdgpu_buffer_rsrc_t wrs = make_rsrc(a.packed[term] + (e * a.N + n0) * a.Kp, rows_here * a.Kp);
    const __amdgpu_buffer_rsrc_t srs = make_rsrc((const unsigned char*)a.w_scale[term] + (e * a.N + n0) * a.G * SB, rows_here * a.G * SB);
    const unsigned woff = (unsigned)r16 * (unsigned)a.Kp + 16u * b;
    const unsigned soff = (unsigned)r16 * (unsigned)a.G * SB;
    // SL: the scales of the workgroup's rows (all of K, one term) are copied into LDS once, as full cache
    // lines; read row by row from global memory, every 16-byte piece would be an L1 miss of its own.
    const unsigned stile = corr_base + (unsigned)((KC / 128) * 16 * MT * 4);
    const unsigned slane = stile + (unsigned)((wave * 16 * R + r16) * (int)a.G * SB);
    auto stage_scales = [&]() {
      const int64_t wg_row0 = (int64_t)blockIdx.x * (WAVES * 16 * R);
      const int64_t wg_rows = a.N - wg_row0 < WAVES * 16 * R ? a.N - wg_row0 : WAVES * 16 * R;
      const unsigned char* src = (const unsigned char*)a.w_scale[term] + (e * a.N + wg_row0) * a.G * SB;
      const int units16 = (int)(wg_rows * a.G * SB / 16);
      if (term > 0) __syncthreads();  // the previous term's scales are no longer read
      for (int u = threadIdx.x; u < units16; u += THREADS) *(lds_u32x4*)(stile + 16 * u) = *(const u32x4*)(src + 16 * (int64_t)u);
      __syncthreads();
    };
    // Ring of PF steps of packed weights in flight per row sub-tile: with ~4 us of loaded HBM latency a CU
    // needs > 100 KiB of requests outstanding to stream at full rate (16 waves x PF x R KiB here).
    constexpr int PF = ABL >= 100 ? 8 : 4;  // (8: timing experiments only; needs K % 2048 == 0 and 2-byte scales)
    constexpr int AB = ABL % 10, AB2 = ABL / 10 % 10;  // up to two ablations at once
    u32x4 ring[PF][R] = {};
    u32x4 sraw[R][2], snext[R][2];  // 8 scales (4 steps) per row sub-tile, and the next 8
    auto fetch_w = [&](int c, u32x4 (&dst)[R]) {
      const int cc = c < steps ? c : steps - 1;  // past the end: re-read the last step, no branch
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (AB == 5 || AB2 == 5) { asm volatile("" : "+v"(dst[r])); continue; }  // ablation: no weight traffic
        dst[r] = buf_load16(wrs, woff, (unsigned)(row_shift[r] * a.Kp) + 64u * cc);
      }
    };
    auto fetch_s = [&](int c, u32x4 (&dst)[R][2]) {  // scales of steps c .. c+3 (c % 4 == 0)
      const int cc = c < steps ? c : 0;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const unsigned so = (unsigned)(row_shift[r] * a.G + ((2 * cc) >> gs)) * SB;
        if (SL) {
          dst[r][0] = *(const lds_u32x4*)(slane + so);
          if (SDT == BP_F32 || PF == 8) dst[r][1] = *(const lds_u32x4*)(slane + so + 16);
          continue;
        }
        dst[r][0] = buf_load16(srs, soff, so);
        if (SDT == BP_F32 || PF == 8) dst[r][1] = buf_load16(srs, soff, so + 16);
      }
    };
    const bool restage = term == 0 || chunks > 1;  // a tile that holds all of K is staged once for all terms
    if (restage) stage_load(0);
    // Same issue order as inside the loop (scales, then the weights step by step), pinned with scheduling
    // barriers: loads return in order, so the loop's waits can then leave the younger loads in flight.
    if (!SL) fetch_s(0, snext);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < PF; ++i) {
      fetch_w(i, ring[i]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (SL) {  // behind the loads above, so that their latencies overlap with the copy's
      stage_scales();
      fetch_s(0, snext);
    }
    for (int ch = 0; ch < chunks; ++ch) {
      if (restage && !((AB == 6 || AB2 == 6) && ch > 0)) {  // (ablation 6: the tile is staged once, results are wrong)
        __syncthreads();  // every wave is done reading the previous tile
        stage_store();
        __syncthreads();
        if (ch + 1 < chunks) stage_load((int64_t)(ch + 1) * KC);
      }
      const int c_end = (ch + 1) * steps_per_chunk < steps ? (ch + 1) * steps_per_chunk : steps;
      for (int c4 = ch * steps_per_chunk; c4 < c_end; c4 += PF) {  // blocks of 4 steps; KC % 1024 == 0 unless the tile holds all of K
#pragma unroll
        for (int r = 0; r < R; ++r) { sraw[r][0] = snext[r][0]; sraw[r][1] = snext[r][1]; }
        fetch_s(c4 + PF, snext);
#pragma unroll
        for (int i = 0; i < PF; ++i) {
          // One scheduling region per step: the wait for this step's weights stays here instead of joining
          // the waits of the later steps at the top of the block.
          __builtin_amdgcn_sched_barrier(0);
          const int c = c4 + i;
          u32x4 w[R];
#pragma unroll
          for (int r = 0; r < R; ++r) {  // regroup: .x/.y = 8 bytes of group 2c, .z/.w = 8 bytes of group 2c+1
            const auto s0 = __builtin_amdgcn_permlane32_swap(ring[i][r].x, ring[i][r].z, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(ring[i][r].y, ring[i][r].w, false, false);
            w[r] = u32x4{s0[0], s1[0], s0[1], s1[1]};
          }
          const int gl = (c - ch * steps_per_chunk) * 2;  // first of the step's two groups within the tile
          const unsigned xoff = (unsigned)(gl * 128 * XB);
          if (AB == 1) {  // ablation (timing experiments only): memory traffic without decode and MFMA
            fetch_w(c + PF, ring[i]);
#pragma unroll
            for (int r = 0; r < R; ++r) total[r][0][0] += __uint_as_float((w[r].x ^ w[r].y ^ w[r].z ^ w[r].w) & 0x3fffffu);
            continue;
          }
          if (c < steps)  // K % 1024 != 0: the last block of 4 steps is partial (the ring re-read the last step)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            typedef typename Acc<ACT>::type acc_t;
            u32x4 xa[NJ][MT];
            acc_t base[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              if (AB == 3 || AB2 == 3) {  // ablation: no LDS operand reads
                base[mt] = acc_t{0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < NJ; ++j) xa[j][mt] = u32x4{kc.M1, kc.M2, kc.M1, kc.M2};
                continue;
              }
              base[mt] = __builtin_bit_cast(acc_t, *(const lds_u32x4*)(corr_lane + ((gl + h) * (16 * MT) + 16 * mt) * 4));
#pragma unroll
              for (int j = 0; j < NJ; ++j) xa[j][mt] = *(const lds_u32x4*)(xaddr[mt] + xoff + (h * 128 + j * KM) * XB);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const unsigned lo = h == 0 ? w[r].x : w[r].z, hi = h == 0 ? w[r].y : w[r].w;
              u32x4 wb[NJ];
              if (AB == 4 || AB2 == 4) {  // ablation: no decode
#pragma unroll
                for (int j = 0; j < NJ; ++j) wb[j] = u32x4{lo, hi, lo | kc.M1, hi | kc.M1};
              } else if (ACT == BP_BF16) {
                tq2_decode_bf16(lo, kc, wb[0], wb[1]);
                tq2_decode_bf16(hi, kc, wb[NJ - 2], wb[NJ - 1]);
              } else {
                wb[0] = tq2_decode_i8(lo);
                wb[1] = tq2_decode_i8(hi);
              }
              // group 2c + h = entry 2i + h of the 8 held (scale groups of 256: one scale per step, entry i)
              const float s_step = scale_at<SDT>(sraw[r], i), s_group = scale_at<SDT>(sraw[r], 2 * i + h);  // (both with constant indices)
              const float s = gs ? s_step : s_group;
#pragma unroll
              for (int mt = 0; mt < MT; ++mt) {
                acc_t acc = base[mt];
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                  if (AB == 2 || AB2 == 2) {  // ablation: operands are produced but no MFMA is issued
                    asm volatile("" ::"v"(xa[j][mt]), "v"(wb[j]));
                    continue;
                  }
                  if (ACT == BP_BF16)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[j][mt]),
                                                                  __builtin_bit_cast(bf16x8, wb[j]), acc, 0, 0, 0);
                  else
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, xa[j][mt]),
                                                                __builtin_bit_cast(i32x4, wb[j]), acc, 0, 0, 0);
                }
#pragma unroll
                for (int q = 0; q < NQ; ++q) total[r][mt][q] += (float)acc[q] * s;
              }
            }
          }
          // Ring slots are reloaded once consumed (in place: no register copies), two steps at a time and
          // back to back: the two 64-byte halves of every 128-byte line then reach the L1 together and go
          // to L2 as one request instead of two that each occupy a miss slot for the full latency.
          __builtin_amdgcn_sched_barrier(0);
          if (i & 1) {
            fetch_w(c - 1 + PF, ring[i - 1]);
            fetch_w(c + PF, ring[i]);
          }
        }
      }
    }
  }
  // ---- epilogue: lane holds tokens 4b + q (q = 0..3) of each token tile, output row n0 + 16r + r16
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int q = 0; q < NQ; ++q) {  // NQ = 1: single-token launches keep only the sums of token 0
      const int t = 16 * mt + 4 * b + q;
      if (t < ntok) {
        const int64_t tok = tok0 + t;
        const float xs = ACT == BP_I8 ? a.x_scale[tok] : 1.0f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (rows_valid[r]) {
            float* o = a.out + tok * a.N + n0 + 16 * r + r16;
            *o += total[r][mt][q] * xs;
          }
        }
      }
    }
  }
}

template <int ACT, int SDT, int R, int MT, int WAVES, int XKB, int ABL = 0, int NQ = 4, int SL = 1>
int launch_tq2(const GemmArgs& a, hipStream_t s, const char* name) {
  constexpr int XB = ACT == BP_BF16 ? 2 : 1;
  const int64_t rows_per_wg = (int64_t)WAVES * 16 * R;
  const dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), (unsigned)a.E,
                  (unsigned)((a.max_rows + 16 * MT - 1) / (16 * MT)));
  // chunk length: as much of K as the tile budget holds for the widest token tile, in blocks of 4 steps
  const int64_t tokens = a.max_rows < 16 * MT ? a.max_rows : 16 * MT;
  // bytes per k: the tokens' activations plus 16 * MT offset sums of 4 bytes per 128-wide group
  int64_t kc = 2 * (XKB * 1024 - 16 * tokens) / (2 * tokens * XB + MT) / 1024 * 1024;
  if (kc > a.K) kc = a.K;
  if (kc < 1024) return fail(BP_ERR_UNSUPPORTED, "activation tile does not fit");
  const size_t stile = SL ? (size_t)rows_per_wg * a.G * (SDT == BP_F32 ? 4 : 2) : 0;
  const size_t lds = X_BASE + (size_t)tokens * (kc * XB + 16) + (size_t)(kc / 128) * 16 * MT * 4 + stile;
  constexpr int lds_want = X_BASE + XKB * 1024 + (SL ? tq2_scale_tile_max(R) : 0);
  constexpr int lds_cap = lds_want < 160 * 1024 ? lds_want : 160 * 1024;
  if (lds > (size_t)lds_cap) return BP_ERR_UNSUPPORTED;  // (scale tile variant: the caller falls back to scales from global memory)
  if (const int rc = raise_lds_limit<k_mfma_tq2<ACT, SDT, R, MT, WAVES, XKB, ABL, NQ, SL>>(lds_cap)) return rc;
  note_kernel(name);
  hipLaunchKernelGGL((k_mfma_tq2<ACT, SDT, R, MT, WAVES, XKB, ABL, NQ, SL>), grid, dim3(WAVES * 64), lds, s, a, (int)kc, (int)tokens);
  return check_launch(name);
}

template <int ACT, int R, int MT, int WAVES, int XKB, int NQ = 4>
int launch_tq2_sd(const GemmArgs& a, hipStream_t s, const char* name) {
  // scales through LDS whenever the workgroup's share of one term fits the budget
  const int64_t tile = (int64_t)WAVES * 16 * R * a.G * (a.scale_dtype == BP_F32 ? 4 : 2);
  // (the tile is read 16 bytes at a time from a row's start + 4 c: rows must be 16 bytes apart modulo 16)
  if (tile <= tq2_scale_tile_max(R) && (a.G * (a.scale_dtype == BP_F32 ? 4 : 2)) % 16 == 0 && a.group == 128) {
    int rc;
    if (a.scale_dtype == BP_F16) rc = launch_tq2<ACT, BP_F16, R, MT, WAVES, XKB, 0, NQ, 1>(a, s, name);
    else if (a.scale_dtype == BP_BF16) rc = launch_tq2<ACT, BP_BF16, R, MT, WAVES, XKB, 0, NQ, 1>(a, s, name);
    else rc = launch_tq2<ACT, BP_F32, R, MT, WAVES, XKB, 0, NQ, 1>(a, s, name);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  if (a.scale_dtype == BP_F16) return launch_tq2<ACT, BP_F16, R, MT, WAVES, XKB, 0, NQ, 0>(a, s, name);
  if (a.scale_dtype == BP_BF16) return launch_tq2<ACT, BP_BF16, R, MT, WAVES, XKB, 0, NQ, 0>(a, s, name);
  return launch_tq2<ACT, BP_F32, R, MT, WAVES, XKB, 0, NQ, 0>(a, s, name);
}

}  // namespace

int launch_mfma_tq2(const GemmArgs& a, hipStream_t s, int R, int MT, int waves) {
  const bool bf = a.x_dtype == BP_BF16;
#ifdef BP_DEV_ABLATIONS  // timing ablations (results are wrong): development builds only
  if (const char* t = getenv("BP_TUNE_ABL")) {
    if (bf && a.scale_dtype == BP_F16 && MT == 1) {
      switch (atoi(t)) {
        case 1: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 1>(a, s, "abl1_w16");
        case 2: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 2>(a, s, "abl2_w16");
        case 3: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 3>(a, s, "abl3_w16");
        case 4: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 4>(a, s, "abl4_w16");
        case 5: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 5>(a, s, "abl5_w16");
        case 25: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 25>(a, s, "abl25_w16");
        case 35: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 35>(a, s, "abl35_w16");
        case 45: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 45>(a, s, "abl45_w16");
        case 100: return launch_tq2<BP_BF16, BP_F16, 1, 1, 16, 48, 100>(a, s, "abl100_w16");
        default: break;
      }
    }
  }
#endif
  if (a.max_rows == 1 && R == 2 && MT == 1 && waves == 16) {
    if (bf) return launch_tq2_sd<BP_BF16, 2, 1, 16, 48, 1>(a, s, "mfma_tq2_bf16_r2_t1_w16");
    return launch_tq2_sd<BP_I8, 2, 1, 16, 48, 1>(a, s, "mfma_tq2_i8_r2_t1_w16");
  }
  if (a.max_rows == 1 && R == 1 && MT == 1) {  // decode GEMV: one token, only its sums are scaled and kept
    if (bf) {
      if (waves == 16) return launch_tq2_sd<BP_BF16, 1, 1, 16, 48, 1>(a, s, "mfma_tq2_bf16_r1_t1_w16");
      return launch_tq2_sd<BP_BF16, 1, 1, 8, 48, 1>(a, s, "mfma_tq2_bf16_r1_t1_w8");
    }
    if (waves == 16) return launch_tq2_sd<BP_I8, 1, 1, 16, 48, 1>(a, s, "mfma_tq2_i8_r1_t1_w16");
    return launch_tq2_sd<BP_I8, 1, 1, 8, 48, 1>(a, s, "mfma_tq2_i8_r1_t1_w8");
  }
#define BP_CASE(ACTV, RV, MTV, WV, XK, NAME) \
  if (R == RV && MT == MTV && waves == WV) return launch_tq2_sd<ACTV, RV, MTV, WV, XK>(a, s, NAME "_r" #RV "_m" #MTV "_w" #WV);
#define BP_ALL(ACTV, NAME)                                                        \
  BP_CASE(ACTV, 1, 1, 8, 48, NAME) BP_CASE(ACTV, 2, 1, 8, 48, NAME)                \
  BP_CASE(ACTV, 1, 1, 16, 48, NAME) BP_CASE(ACTV, 2, 1, 16, 48, NAME)
  if (bf) { BP_ALL(BP_BF16, "mfma_tq2_bf16") } else { BP_ALL(BP_I8, "mfma_tq2_i8") }
#undef BP_ALL
#undef BP_CASE
  return fail(BP_ERR_UNSUPPORTED, "no tuned kernel variant for this tiling");
}

}  // namespace bp

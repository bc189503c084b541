// TQ2 grouped GEMM for token tiles of 32 rows (prefill, routed experts with many tokens each).
//
// Same arithmetic as bp_mfma_tq2.hip (table-free decode into MFMA operands, offsets removed through the
// accumulator's start value, scale applied per 128-wide group), organised for the regime where the matrix
// cores and the LDS, not HBM, set the pace:
//  * 8 waves per workgroup, two 16-row sub-tiles per wave: the decoded weights of a lane meet 32 tokens,
//    and every activation operand read from LDS feeds two MFMAs. Two waves per SIMD leave each wave 256
//    registers.
//  * The activation tile is stored fragment-major: the 64 x 16 bytes that one MFMA takes as operand A are
//    one contiguous KiB in lane order, so an operand read is conflict-free (a token-major tile with a
//    padded pitch costs 1.6x the LDS time of this layout on gfx950).
//  * Two activation tiles in LDS: the next 1024 k are loaded to registers while the current tile is
//    multiplied and stored when it ends, with one barrier per tile.
//  * Workgroups that share an expert's activations run on the same XCD (one L2).
#include <type_traits>

#include "bp_mfma.h"
#include "bp_tq2_decode.h"

namespace bp {
namespace {

constexpr int GW = 8;               // waves per workgroup
constexpr int GR = 2;               // 16-row sub-tiles per wave
constexpr int GT = 2;               // 16-token sub-tiles per workgroup
constexpr int GKC = 1024;           // k per activation tile: 8 groups, 4 steps of 64 packed bytes
constexpr int GTHREADS = GW * 64;
constexpr int GROWS = GW * 16 * GR;  // output rows per workgroup
constexpr int GCORR = (GKC / 128) * 16 * GT * 4;  // bytes of offset sums per tile

template <int ACT>
constexpr int gemm_tile_bytes() { return 16 * GT * GKC * (ACT == BP_BF16 ? 2 : 1) + GCORR; }

// LDS: 2 x (fragments | offset sums) | scale tile.
// Fragment (g, j, mt) of a tile - group g of 8, MFMA j of NJ within the group, token sub-tile mt - is the
// KiB at ((g * NJ + j) * GT + mt) * 1024; lane l = 16 b + t of it holds, for token 16 mt + t, the KM
// elements the lane multiplies in that MFMA (k-block b of the decode's slot order).
template <int ACT, int SDT, int SL, int ABL = 0>
__global__ __launch_bounds__(GTHREADS, 2) void k_gemm_tq2(GemmArgs a) {
  constexpr int XB = ACT == BP_BF16 ? 2 : 1;
  constexpr int KM = ACT == BP_BF16 ? 8 : 16;
  constexpr int NJ = 32 / KM;
  constexpr int TILE = gemm_tile_bytes<ACT>();
  constexpr int XT = TILE - GCORR;
  constexpr int SB = SDT == BP_F32 ? 4 : 2;
  constexpr int PF = 4;  // steps per activation tile
  constexpr int RD = 4;  // steps of packed weights in flight per row sub-tile
  static_assert(16 * (GKC / 32) == GTHREADS, "one staging item (32 elements of one token) per thread and token sub-tile");
  typedef typename Acc<ACT>::type acc_t;

  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, b = lane >> 4;
  const int row_tiles = (int)((a.N + GROWS - 1) / GROWS);
  int wg_tile;
  const TileRef tr = tile_of_workgroup(a, blockIdx.x, row_tiles, wg_tile);
  if (!tr.live) return;  // uniform for the workgroup
  const int64_t e = tr.e, tok0 = tr.tok0, o1 = tr.o1;
  const int ntok = (int)(o1 - tok0 < 16 * GT ? o1 - tok0 : 16 * GT);
  const bool two = ntok > 16;  // the second token sub-tile holds tokens
  int64_t n0 = ((int64_t)wg_tile * GW + wave) * (16 * GR);
  const bool wave_live = n0 < a.N;
  if (!wave_live) n0 = 0;
  bool rows_valid[GR];
  int64_t row_shift[GR];
#pragma unroll
  for (int r = 0; r < GR; ++r) {
    rows_valid[r] = wave_live && n0 + 16 * r < a.N;
    row_shift[r] = rows_valid[r] ? 16 * r : 0;
  }

  const int chunks = (int)((a.K + GKC - 1) / GKC);  // K % 256 == 0: the last tile may hold 1 to 3 steps only
  // ---- activation staging: thread = (token t of 16, quarter q of a group, group g = wave), once per sub-tile
  const int sq = (lane >> 4), sg = wave;
  const int sb = ((sq & 1) << 1) | (sq >> 1);  // k-block that holds elements 32 q .. 32 q + 31 of a group
  const unsigned char* xg = (const unsigned char*)a.x + tok0 * a.K * XB;
  // The thread's share of the next tile (one item per token sub-tile) is loaded when the current tile starts
  // and stored to the other LDS tile when it ends: a whole tile time hides the load latency.
  // Loads: an instruction reads, per token row, the four 16-byte pieces of a 64-byte segment with four
  // lanes (16 rows x 64 B: 16 memory requests; one lane per 64-byte item would make 64). bf16: a 16-element
  // permutation unit is two pieces; lanes l and l + 32 hold the two pieces of a unit and trade them with
  // v_permlane32_swap, the lower half of the wave ending with the units of one segment, the upper half
  // with those of the next.
  u32x4 xsr[GT][2][XB];
  auto stage_load = [&](int64_t k0, int mt) {
    if (mt == 1 && !two) return;
    if (k0 + sg * 128 >= a.K) return;  // (last tile: this wave's group lies past K; its part of the tile is never read)
    auto& xs = xsr[mt];
    int row = 16 * mt + r16;
    if (row >= ntok) row = ntok - 1;
    const unsigned char* p = xg + ((int64_t)row * a.K + k0 + sg * 128) * XB;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      if (ACT == BP_BF16) {
#pragma unroll
        for (int v = 0; v < XB; ++v) xs[e][v] = *(const u32x4*)(p + (2 * e + v) * 64 + sb * 16);
      } else {
        xs[e][0] = *(const u32x4*)(p + e * 64 + sq * 16);
      }
    }
  };
  // sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 with row swaps in the vector ALU (a shuffle through the
  // LDS pipeline would wait behind the operand reads of all the other waves)
  auto sum4 = [](unsigned v, bool is_float) {
    auto add = [&](unsigned x, unsigned y) { return is_float ? __float_as_uint(__uint_as_float(x) + __uint_as_float(y)) : x + y; };
    const auto r16 = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    const unsigned s = add(r16[0], r16[1]);
    const auto r32 = __builtin_amdgcn_permlane32_swap(s, s, false, false);
    return add(r32[0], r32[1]);
  };
  auto stage_store = [&](int buf, int mt) {
    if (mt == 1 && !two) return;
    auto& xs = xsr[mt];
    const unsigned tile = (unsigned)(buf * TILE);
    unsigned part;
    float f = 0.f;
    int n = 0;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      // this lane's unit: the (4 e + sq)-th 16 elements of group sg -> MFMA j0 (and j0 + 1), k-block kb
      const int c = 4 * e + sq;
      if (ACT == BP_BF16) {
        u32x4 ua, uc;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const auto r = __builtin_amdgcn_permlane32_swap(xs[e][0][d], xs[e][XB - 1][d], false, false);
          ua[d] = r[0];
          uc[d] = r[1];
        }
        const int q = c >> 1, kb = ((q & 1) << 1) | (q >> 1);
        const unsigned dst = tile + (unsigned)(((sg * NJ + 2 * (c & 1)) * GT + mt) * 1024 + (kb * 16 + r16) * 16);
        u32x4 p0, p1;
        tq2_permute_bf16(ua, uc, p0, p1);
        *(lds_u32x4*)(dst) = p0;
        *(lds_u32x4*)(dst + GT * 1024) = p1;
        const bf16x2 w93 = __builtin_bit_cast(bf16x2, 0x40404110u);  // (9.0, 3.0): even k in the low half
        const unsigned dw[8] = {ua.x, ua.y, ua.z, ua.w, uc.x, uc.y, uc.z, uc.w};
#pragma unroll
        for (int d = 0; d < 8; ++d) f = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, dw[d]), w93, f, false);
      } else {
        const int q = c >> 1, kb = ((q & 1) << 1) | (q >> 1);
        const unsigned dst = tile + (unsigned)(((sg * NJ + (c & 1)) * GT + mt) * 1024 + (kb * 16 + r16) * 16);
        *(lds_u32x4*)(dst) = tq2_permute_i8(xs[e][0]);
        const unsigned dw[4] = {xs[e][0].x, xs[e][0].y, xs[e][0].z, xs[e][0].w};
#pragma unroll
        for (int d = 0; d < 4; ++d) n = __builtin_amdgcn_sdot4((int)dw[d], 0x01010101, n, false);
      }
    }
    if (ACT == BP_BF16) {
      part = __float_as_uint(-__uint_as_float(sum4(__float_as_uint(f), true)));
    } else {
      part = (unsigned)(-(int)sum4((unsigned)n, false));
    }
    if (sq == 0) *(lds_u32*)(tile + XT + (sg * (16 * GT) + 16 * mt + r16) * 4) = part;
  };
  auto tile_k0 = [&](int t) { return (int64_t)(t % chunks) * GKC; };

  f32x4 total[GR][GT];
#pragma unroll
  for (int r = 0; r < GR; ++r)
#pragma unroll
    for (int mt = 0; mt < GT; ++mt) total[r][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  Tq2Consts kc = {0x00c000c0u, 0x00300030u, 0x40004000u, 0x41004100u};
  asm volatile("" : "+s"(kc.P1), "+s"(kc.P2));
  asm volatile("" : "+v"(kc.M1), "+v"(kc.M2));

  const int steps = (int)(a.K / 256);
  const int gs = a.group == 256 ? 1 : 0;  // scale groups of 256: the two 128-wide halves of a step share a scale (read from global memory)
  const int tiles = chunks == 1 ? 1 : a.n_terms * chunks;  // activation tiles to stage (one tile serves all terms)
  const unsigned stile = (unsigned)(2 * TILE);
  const unsigned xlane = (unsigned)(lane * 16);
  const unsigned clane = (unsigned)(XT + 16 * b);

  // first tile: its loads are issued here, ahead of the first term's weight and scale loads, and stored once those
  // are on their way too (one memory latency for all of them)
  stage_load(0, 0);
  stage_load(0, 1);
  int seq = 0;  // tiles consumed so far
  // The whole loop nest is instantiated once per number of token sub-tiles and the choice made outside it: a branch
  // inside would end in a merge of the two paths' registers, and a register that a load in flight is about to write
  // can only be merged after waiting for that load - the weight ring would drain at the end of every tile.
  auto all_terms = [&](auto mtn_c) {
  u32x4 ring[RD][GR];
  constexpr int SPRE = 4;  // 16-byte units of the scale tile per thread that are fetched ahead (the rest, if any, at the term's start)
  u32x4 spre[SPRE];
  bool ring_filled = false;  // the ring already holds the term's first steps (loaded at the end of the term before)
  for (int term = 0; term < a.n_terms; ++term) {
    const int64_t rows_here = a.N - n0 < 16 * GR ? a.N - n0 : 16 * GR;
    const __amdgpu_buffer_rsrc_t wrs = make_rsrc(a.packed[term] + (e * a.N + n0) * a.Kp, rows_here * a.Kp);
    // a term's last refills of the ring run on into the next term's first steps (whole tiles only: the ring slot of a
    // step is its index within the tile)
    const bool chain = steps % PF == 0 && term + 1 < a.n_terms;
    const __amdgpu_buffer_rsrc_t wrs_next = make_rsrc(a.packed[chain ? term + 1 : term] + (e * a.N + n0) * a.Kp, rows_here * a.Kp);
    const __amdgpu_buffer_rsrc_t srs = make_rsrc((const unsigned char*)a.w_scale[term] + (e * a.N + n0) * a.G * SB, rows_here * a.G * SB);
    const unsigned woff = (unsigned)r16 * (unsigned)a.Kp + 16u * b;
    const unsigned soff = (unsigned)r16 * (unsigned)a.G * SB;
    const unsigned slane = stile + (unsigned)((wave * 16 * GR + r16) * (int)a.G * SB);
    u32x4 sraw[GR][2], snext[GR][2];
    auto fetch_w = [&](int c, u32x4 (&dst)[GR]) {
      const bool over = chain && c >= steps;
      const int cc = over ? c - steps : c < steps ? c : steps - 1;
#pragma unroll
      for (int r = 0; r < GR; ++r) {
        if (ABL == 5) { asm volatile("" : "+v"(dst[r])); continue; }
        dst[r] = buf_load16(over ? wrs_next : wrs, woff, (unsigned)(row_shift[r] * a.Kp) + 64u * cc);
      }
    };
    auto fetch_s = [&](int c, u32x4 (&dst)[GR][2]) {  // scales of steps c .. c+3
      const int cc = c < steps ? c : 0;
#pragma unroll
      for (int r = 0; r < GR; ++r) {
        const unsigned so = (unsigned)(row_shift[r] * a.G + ((2 * cc) >> gs)) * SB;
        if (SL) {
          dst[r][0] = *(const lds_u32x4*)(slane + so);
          if (SDT == BP_F32) dst[r][1] = *(const lds_u32x4*)(slane + so + 16);
        } else {
          dst[r][0] = buf_load16(srs, soff, so);
          if (SDT == BP_F32) dst[r][1] = buf_load16(srs, soff, so + 16);
        }
      }
    };
    // the workgroup's rows of a term's scales: one contiguous block, copied to LDS in 16-byte units
    const int64_t wg_row0 = (int64_t)wg_tile * GROWS;
    const int64_t wg_rows = a.N - wg_row0 < GROWS ? a.N - wg_row0 : GROWS;
    const int units16 = (int)(wg_rows * a.G * SB / 16);
    auto scale_prefetch = [&](int t) {
      const unsigned char* src = (const unsigned char*)a.w_scale[t] + (e * a.N + wg_row0) * a.G * SB;
#pragma unroll
      for (int i = 0; i < SPRE; ++i) {
        const int u = (int)threadIdx.x + i * GTHREADS;
        if (u < units16) spre[i] = *(const u32x4*)(src + 16 * (int64_t)u);
      }
    };
    if (!SL) fetch_s(0, snext);
    __builtin_amdgcn_sched_barrier(0);
    if (!ring_filled) {
#pragma unroll
      for (int i = 0; i < RD; ++i) {
        fetch_w(i, ring[i]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    ring_filled = chain;
    if (SL) {
      if (term == 0) scale_prefetch(0);
      else __syncthreads();  // the previous term's scales are no longer read
#pragma unroll
      for (int i = 0; i < SPRE; ++i) {
        const int u = (int)threadIdx.x + i * GTHREADS;
        if (u < units16) *(lds_u32x4*)(stile + 16 * u) = spre[i];
      }
      const unsigned char* src = (const unsigned char*)a.w_scale[term] + (e * a.N + wg_row0) * a.G * SB;
      for (int u = threadIdx.x + SPRE * GTHREADS; u < units16; u += GTHREADS) *(lds_u32x4*)(stile + 16 * u) = *(const u32x4*)(src + 16 * (int64_t)u);
    }
    if (term == 0) {
      stage_store(0, 0);
      stage_store(0, 1);
      if (tiles > 1) {
        stage_load(tile_k0(1), 0);
        stage_load(tile_k0(1), 1);
      }
    }
    if (SL || term == 0) __syncthreads();
    if (SL) fetch_s(0, snext);

    for (int ch = 0; ch < chunks; ++ch) {
      // a tile that holds all of K is staged once and serves every term
      const bool staged = (chunks > 1 || term == 0) && !(ABL == 6 && seq > 0);
      const int buf = chunks > 1 ? (seq & 1) : 0;
      const bool more = staged && seq + 1 < tiles;
      const unsigned xbase = (unsigned)(buf * TILE) + xlane;
      const unsigned cbase = (unsigned)(buf * TILE) + clane;

#pragma unroll
      for (int r = 0; r < GR; ++r) { sraw[r][0] = snext[r][0]; sraw[r][1] = snext[r][1]; }
      const int c4 = ch * PF;
      fetch_s(c4 + PF, snext);
      if (SL && ch == chunks - 1 && term + 1 < a.n_terms) scale_prefetch(term + 1);

      // The four steps of the tile, for MTN token sub-tiles (a tile of at most 16 tokens skips the second one).
      auto run_steps = [&](auto mtn_c) {
        constexpr int MTN = decltype(mtn_c)::value;
        // One group's operands at a time; the compiler hoists these reads ahead of the previous group's MFMAs as
        // far as registers allow (an explicit second operand buffer costs 40 registers and spills the staging data).
        u32x4 xa[NJ][GT];
        acc_t base[GT];
        auto load_x = [&](int gl, u32x4 (&dx)[NJ][GT], acc_t (&db)[GT]) {
#pragma unroll
          for (int mt = 0; mt < MTN; ++mt) {
            if (ABL == 3) {
              db[mt] = acc_t{0, 0, 0, 0};
#pragma unroll
              for (int j = 0; j < NJ; ++j) dx[j][mt] = u32x4{kc.M1, kc.M2, kc.M1, kc.M2};
              continue;
            }
            db[mt] = __builtin_bit_cast(acc_t, *(const lds_u32x4*)(cbase + (gl * (16 * GT) + 16 * mt) * 4));
#pragma unroll
            for (int j = 0; j < NJ; ++j) dx[j][mt] = *(const lds_u32x4*)(xbase + ((gl * NJ + j) * GT + mt) * 1024);
          }
        };
#pragma unroll
        for (int i = 0; i < PF; ++i) {
          __builtin_amdgcn_sched_barrier(0);
          const int c = c4 + i;
          u32x4 w[GR];
#pragma unroll
          for (int r = 0; r < GR; ++r) {  // regroup: .x/.y = 8 bytes of group 2c, .z/.w = 8 bytes of group 2c+1
            const auto s0 = __builtin_amdgcn_permlane32_swap(ring[i % RD][r].x, ring[i % RD][r].z, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(ring[i % RD][r].y, ring[i % RD][r].w, false, false);
            w[r] = u32x4{s0[0], s1[0], s0[1], s1[1]};
          }
          if (c < steps)  // (K % 1024 != 0: the last tile ends early)
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int gl = 2 * i + h;
            load_x(gl, xa, base);
#pragma unroll
            for (int r = 0; r < GR; ++r) {
              const unsigned lo = h == 0 ? w[r].x : w[r].z, hi = h == 0 ? w[r].y : w[r].w;
              u32x4 wb[NJ];
              if (ABL == 4) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) wb[j] = u32x4{lo, hi, lo | kc.M1, hi | kc.M1};
              } else if (ACT == BP_BF16) {
                tq2_decode_bf16(lo, kc, wb[0], wb[1]);
                tq2_decode_bf16(hi, kc, wb[NJ - 2], wb[NJ - 1]);
              } else {
                wb[0] = tq2_decode_i8(lo);
                wb[1] = tq2_decode_i8(hi);
              }
              // (scale groups of 256: one scale per step; both candidates are read with constant indices)
            const float s_step = scale_at<SDT>(sraw[r], i), s_group = scale_at<SDT>(sraw[r], 2 * i + h);
            const float s = gs ? s_step : s_group;
              acc_t acc[GT];
#pragma unroll
              for (int mt = 0; mt < MTN; ++mt) acc[mt] = base[mt];
#pragma unroll
              for (int j = 0; j < NJ; ++j) {  // the two token sub-tiles alternate: no MFMA waits on the one before it
#pragma unroll
                for (int mt = 0; mt < MTN; ++mt) {
                  if (ACT == BP_BF16)
                    acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[j][mt]),
                                                                      __builtin_bit_cast(bf16x8, wb[j]), acc[mt], 0, 0, 0);
                  else
                    acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, xa[j][mt]),
                                                                    __builtin_bit_cast(i32x4, wb[j]), acc[mt], 0, 0, 0);
                }
              }
#pragma unroll
              for (int mt = 0; mt < MTN; ++mt) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  if (ABL == 7) { if (q == 0) total[r][mt][0] += (float)(acc[mt][0] + acc[mt][1] + acc[mt][2] + acc[mt][3]) * s; continue; }
                  total[r][mt][q] += (float)acc[mt][q] * s;
                }
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);
          if (i & 1) {  // reload the consumed ring slots in place, two steps back to back (whole 128-byte lines)
            fetch_w(c - 1 + RD, ring[(i - 1) % RD]);
            fetch_w(c + RD, ring[i % RD]);
          }
        }

      };
      run_steps(mtn_c);

      if (staged) {
        if (more) {
          stage_store(buf ^ 1, 0);  // the other tile: last read before the previous barrier
          stage_store(buf ^ 1, 1);
          if (seq + 2 < tiles) {
            stage_load(tile_k0(seq + 2), 0);
            stage_load(tile_k0(seq + 2), 1);
          }
        }
        __syncthreads();
        ++seq;
      }
    }
  }
  };
  if (two) all_terms(std::integral_constant<int, GT>{});
  else all_terms(std::integral_constant<int, 1>{});

  // ---- epilogue: lane holds tokens 4b + q of each token sub-tile, output row n0 + 16r + r16
#pragma unroll
  for (int mt = 0; mt < GT; ++mt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int t = 16 * mt + 4 * b + q;
      if (t < ntok) {
        const int64_t tok = tok0 + t;
        const float xs = ACT == BP_I8 ? a.x_scale[tok] : 1.0f;
#pragma unroll
        for (int r = 0; r < GR; ++r) {
          if (rows_valid[r]) {
            float* o = a.out + tok * a.N + n0 + 16 * r + r16;
            *o = (a.overwrite ? 0.f : *o) + total[r][mt][q] * xs;
          }
        }
      }
    }
  }
}

template <int ACT, int SDT, int SL, int ABL = 0>
int launch_gemm_k(const GemmArgs& a, hipStream_t s, size_t lds, const char* name) {
  if (const int rc = raise_lds_limit<k_gemm_tq2<ACT, SDT, SL, ABL>>(160 * 1024)) return rc;
  static_assert(16 * GT == 32, "tile_of_workgroup counts token tiles of 32");
  const int64_t wgs = tile_workgroups(a, (a.N + GROWS - 1) / GROWS);
  if (wgs < 0) return BP_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)wgs, 1, 1);
  note_kernel(name);
  hipLaunchKernelGGL((k_gemm_tq2<ACT, SDT, SL, ABL>), grid, dim3(GTHREADS), lds, s, a);
  return check_launch(name);
}

// scales through LDS when the workgroup's rows of one term fit beside the two activation tiles
template <int ACT, int SDT>
int launch_gemm_sd(const GemmArgs& a, hipStream_t s, const char* name, const char* name_gs) {
  const size_t tiles = 2 * (size_t)gemm_tile_bytes<ACT>();
  const size_t stile = (size_t)GROWS * a.G * (SDT == BP_F32 ? 4 : 2);
  // (scale tile rows are read 16 bytes at a time: they must start 16-byte aligned)
  if (tiles + stile <= 160 * 1024 && (a.G * (SDT == BP_F32 ? 4 : 2)) % 16 == 0 && a.group == 128) return launch_gemm_k<ACT, SDT, 1>(a, s, tiles + stile, name);
  return launch_gemm_k<ACT, SDT, 0>(a, s, tiles, name_gs);
}

}  // namespace

// Preconditions (checked by mfma_supports): group 128, K % 256 == 0, K >= 1024, N % 16 == 0, 16-byte aligned x / packed / scales.
int launch_gemm_tq2(const GemmArgs& a, hipStream_t s) {
  if (a.stage && tuning().tq2g != 'b') {  // with a workspace: the fp8 x fp4 kernel over converted activations (development: BP_TUNE_TQ2G=bf16 keeps this file's kernel)
    const int rc = launch_gemm_tq2f(a, s);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
#ifdef BP_DEV_ABLATIONS  // timing ablations (results are wrong): development builds only
  if (const char* t = getenv("BP_TUNE_ABL")) {
    const size_t lds = 2 * gemm_tile_bytes<BP_BF16>() + (size_t)GROWS * a.G * 2;
    if (a.x_dtype == BP_BF16 && a.scale_dtype == BP_F16 && lds <= 160 * 1024 && a.K % 1024 == 0 && a.group == 128) {
      switch (atoi(t)) {
        case 2: return launch_gemm_k<BP_BF16, BP_F16, 1, 2>(a, s, lds, "gemm_abl2");
        case 3: return launch_gemm_k<BP_BF16, BP_F16, 1, 3>(a, s, lds, "gemm_abl3");
        case 4: return launch_gemm_k<BP_BF16, BP_F16, 1, 4>(a, s, lds, "gemm_abl4");
        case 5: return launch_gemm_k<BP_BF16, BP_F16, 1, 5>(a, s, lds, "gemm_abl5");
        case 6: return launch_gemm_k<BP_BF16, BP_F16, 1, 6>(a, s, lds, "gemm_abl6");
        case 7: return launch_gemm_k<BP_BF16, BP_F16, 1, 7>(a, s, lds, "gemm_abl7");
        default: break;
      }
    }
  }
#endif
  if (a.x_dtype == BP_BF16) {
    if (a.scale_dtype == BP_F16) return launch_gemm_sd<BP_BF16, BP_F16>(a, s, "gemm_tq2_bf16", "gemm_tq2_bf16_gs");
    if (a.scale_dtype == BP_BF16) return launch_gemm_sd<BP_BF16, BP_BF16>(a, s, "gemm_tq2_bf16", "gemm_tq2_bf16_gs");
    return launch_gemm_sd<BP_BF16, BP_F32>(a, s, "gemm_tq2_bf16", "gemm_tq2_bf16_gs");
  }
  if (a.scale_dtype == BP_F16) return launch_gemm_sd<BP_I8, BP_F16>(a, s, "gemm_tq2_i8", "gemm_tq2_i8_gs");
  if (a.scale_dtype == BP_BF16) return launch_gemm_sd<BP_I8, BP_BF16>(a, s, "gemm_tq2_i8", "gemm_tq2_i8_gs");
  return launch_gemm_sd<BP_I8, BP_F32>(a, s, "gemm_tq2_i8", "gemm_tq2_i8_gs");
}

}  // namespace bp

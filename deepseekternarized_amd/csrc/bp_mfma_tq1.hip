// TQ1 (5 trits per byte, base 3) on MFMA, bf16 or int8 activations. K % 256 == 0, K >= 1024, N % 16 == 0.
// int8 activations are widened to bf16 when the tile is staged (exact: |q| <= 127), so a group's sum of
// q * trit is an exact integer in the float32 accumulator, as in the integer kernels; the token's
// activation scale multiplies the finished sum.
//
// 640 trits = 128 bytes = 5 scale groups realign byte and group boundaries, so the unit of work is a
// 128-byte chunk of every row. A byte is atomic: it fills one MFMA k-block with its 5 trits and 3
// zeros. Group g of a chunk touches bytes FB[g] .. FB[g] + 25 or 26; it is given 28 byte slots
// (7 MFMAs x 4 k-blocks), k-block b of MFMA m taking byte FB[g] + 7 b + m.
//
// Which digits of a byte count for a group is decided on the activation side: the activation tile in
// LDS holds, for every (chunk, group, slot), a 16-byte operand with the 5 activations of that slot's
// byte, zeroed where the digit belongs to a neighbouring group, lies past K, or the slot lies past the
// group's last byte. The weight side is then uniform: every byte decodes in full.
//
// Table entry of byte v: 8 bytes, byte i = high byte of bf16(trit_i / 2) (0x3f, 0xbf or 0), bytes 5..7
// zero; values >= 243 decode to zeros. +-0.5 has a zero low byte, so a v_perm_b32 per operand dword
// expands the entry to bf16; the factor 2 is folded into the group scale (exact).
//
// Packed bytes: every lane loads two aligned 16-byte pieces of its row's 128-byte chunk (plus the dword
// after it) with buffer loads - reads past the end of the tensor return zeros -, the wave transposes
// them through a private LDS buffer and every lane reads back the 7 consecutive bytes of its k-block
// for each group. Two chunks are fetched back to back, so the L1 sees whole 128-byte lines.
#include "bp_mfma.h"

namespace bp {
namespace {

struct __attribute__((packed, aligned(2))) Packed16 { u32x4 v; };
struct __attribute__((packed, aligned(1))) Packed8 { u32x2 v; };

// LDS map: [0, 32 KiB) table, entry of byte v copy c at v * 128 + c * 8; then per wave two row buffers
// of 16 rows x WROW bytes; then the activation tile; then (SL) the workgroup's scales.
constexpr int T1_STRIDE = 128;
constexpr int T1_LUT_BYTES = 256 * T1_STRIDE;
constexpr int T1_SLOTS = 140;                // byte slots per chunk: 5 groups x 28
constexpr int T1_XCHUNK = T1_SLOTS * 16;     // bytes of the activation tile per token and chunk
constexpr int T1_X_BUDGET = 48 * 1024;
constexpr int T1_LDS_MAX = 160 * 1024;
// row pitch of the transpose buffers: 132 bytes of data (+ 12 of scales without the scale tile); a multiple
// of 16 (aligned 16-byte writes) whose 16 rows start in different banks
// (float32 scales without the scale tile: 24 bytes of scales at offset 136)
template <int SL, int SDT>
constexpr int t1_wrow() { return !SL && SDT == BP_F32 ? 160 : 144; }
template <int WAVES, int SL, int SDT>
constexpr int t1_x_base() { return T1_LUT_BYTES + WAVES * 2 * 16 * t1_wrow<SL, SDT>(); }

__device__ __forceinline__ u32x2 buf_load8(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned wave_off) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)lane_off, (int)wave_off, 0));
}

__device__ __forceinline__ unsigned buf_load4(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned wave_off) {
  return (unsigned)__builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, (int)wave_off, 0);
}

// SL: scales through an LDS tile (copied once per workgroup and term) instead of per-chunk loads.
// NQ: token sums kept per lane (4, or 1 for single-token launches).
// MULTI: the activation tile holds only part of K and is restaged inside the chunk loop.
template <int SDT, int WAVES, int NQ, int SL, int MULTI, int ABL = 0>
__global__ __launch_bounds__(WAVES * 64, 4) void k_mfma_tq1(GemmArgs a, int CPT /* chunks per activation tile */, int tile_rows) {
  constexpr int THREADS = WAVES * 64;
  constexpr int WROW = t1_wrow<SL, SDT>();
  constexpr int WB = T1_LUT_BYTES;
  constexpr int XB0 = t1_x_base<WAVES, SL, SDT>();
  constexpr int SB = SDT == BP_F32 ? 4 : 2;  // bytes per scale
  constexpr int XU = (T1_X_BUDGET / 16 + THREADS - 1) / THREADS;  // activation slots staged per thread
  constexpr int FB[5] = {0, 25, 51, 76, 102};

  // ---- table
  if (threadIdx.x < 256) {
    const unsigned v = threadIdx.x;
    unsigned hb[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) { const int t = tq1_trit(v, i); hb[i] = t > 0 ? 0x3fu : t < 0 ? 0xbfu : 0u; }
    const u32x2 e = {hb[0] | (hb[1] << 8) | (hb[2] << 16) | (hb[3] << 24), hb[4]};
    for (int c = 0; c < 16; ++c) *(lds_u32x2*)(v * T1_STRIDE + c * 8) = e;
  }

  // the wave index through readfirstlane: everything derived from it stays in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, b = lane >> 4;
  const int64_t e = blockIdx.y;
  const int64_t o0 = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  const int64_t tok0 = o0 + (int64_t)blockIdx.z * 16;
  if (tok0 >= o1) return;  // uniform for the workgroup
  const int ntok = (int)(o1 - tok0 < 16 ? o1 - tok0 : 16);
  int64_t n0 = ((int64_t)blockIdx.x * WAVES + wave) * 16;
  const bool wave_live = n0 < a.N;
  if (!wave_live) n0 = 0;  // keeps addresses valid; the wave still takes part in staging and barriers
  const unsigned lane_off = (unsigned)(r16 * 8);

  const int nchunks = (int)((a.K + 639) / 640);  // 128-byte chunks per row (the last may be partial)
  const int gs = a.group == 256 ? 1 : 0;         // scale groups of 256: two 128-wide work groups share a scale

  // ---- activation tile: slot (cl, g, 7 b + m) of token t at XB0 + t * pitch + ((cl * 5 + g) * 28 + 7 b + m) * 16
  const int tile_slots = CPT * T1_SLOTS;
  const int pitch = tile_slots * 16 + 16;
  const int units = ntok * tile_slots;
  int t_lane = r16 < ntok ? r16 : ntok - 1;
  const unsigned xaddr = (unsigned)(XB0 + t_lane * pitch + 7 * 16 * b);
  const bool x_i8 = a.x_dtype == BP_I8;  // uniform
  const uint16_t* xg = (const uint16_t*)a.x + tok0 * a.K;
  const signed char* xg8 = (const signed char*)a.x + tok0 * a.K;
  // 16-bit activations are staged without waiting for a load right after issuing it (a wait would also drain the
  // packed bytes in flight): stage_load only requests a slot's activations - 16 raw bytes into the slot's registers -
  // and stage_store, a tile later, picks the slot's 5 values out of them, zeroes the digits of other groups and
  // writes the slot. int8 activations and the last bytes of a row are finished at once.
  u32x4 xstage[XU];
  struct Slot { int row, rem, lo, hi; int64_t k0; bool any, fast; };
  auto slot_of = [&](int u, int chunk0) -> Slot {
    Slot t;
    t.row = u / tile_slots;
    t.rem = u - t.row * tile_slots;
    const int cl = t.rem / T1_SLOTS, sg = t.rem - cl * T1_SLOTS;
    const int g = sg / 28, sl = sg - g * 28;                   // sl = 7 b + m: byte FB[g] + sl of the chunk
    const int j = (g == 0 ? 0 : g == 1 ? 25 : g == 2 ? 51 : g == 3 ? 76 : 102) + sl;
    t.k0 = 640 * (int64_t)(chunk0 + cl) + 5 * j;               // first activation of the byte
    t.lo = 128 * g - 5 * j;                                    // digits lo <= d < hi belong to group g
    t.hi = t.lo + 128;
    if (a.K - t.k0 < t.hi) t.hi = (int)(a.K - t.k0);           // ... and lie inside K
    t.any = t.hi > 0 && t.lo < 5;
    t.fast = t.k0 + 8 <= a.K;
    return t;
  };
  auto finish = [&](const unsigned (&h)[5], const Slot& t) -> u32x4 {  // 5 bf16 patterns -> the slot, other groups' digits zeroed
    unsigned m[5];
#pragma unroll
    for (int d = 0; d < 5; ++d) m[d] = d >= t.lo && d < t.hi ? h[d] : 0u;
    return u32x4{m[0] | (m[1] << 16), m[2] | (m[3] << 16), m[4], 0u};
  };
  auto stage_load = [&](int chunk0) {  // global -> registers: the tile that starts at chunk `chunk0`
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      const int u = threadIdx.x + i * THREADS;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (u < units) {
        const Slot t = slot_of(u, chunk0);
        if (t.any && t.fast && !x_i8) {
          v = ((const Packed16*)(xg + (int64_t)t.row * a.K + t.k0))->v;
        } else if (t.any && t.fast) {  // int8: widened at once (deferring it as well was measured slower)
          const u32x2 q = ((const Packed8*)(xg8 + (int64_t)t.row * a.K + t.k0))->v;
          unsigned h[5];
#pragma unroll
          for (int d = 0; d < 5; ++d) h[d] = __float_as_uint((float)(int)__builtin_amdgcn_sbfe(d < 4 ? q.x : q.y, 8 * (d & 3), 8)) >> 16;  // (the builtin returns unsigned) exact in bf16
          v = finish(h, t);
        } else if (t.any) {  // the last bytes of a row: element by element
          unsigned h[5];
#pragma unroll
          for (int d = 0; d < 5; ++d) {
            if (x_i8) h[d] = t.k0 + d < a.K ? __float_as_uint((float)(int)xg8[(int64_t)t.row * a.K + t.k0 + d]) >> 16 : 0u;  // exact in bf16
            else h[d] = t.k0 + d < a.K ? (unsigned)xg[(int64_t)t.row * a.K + t.k0 + d] : 0u;
          }
          v = finish(h, t);
        }
      }
      xstage[i] = v;
    }
  };
  auto stage_store = [&](int chunk0) {  // registers -> LDS: the tile that starts at chunk `chunk0`, requested by stage_load(chunk0)
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      const int u = threadIdx.x + i * THREADS;
      if (u < units) {
        u32x4 v = xstage[i];
        if (x_i8) {  // (uniform) finished at the load: only the slot's place is needed
          const int row = u / tile_slots, rem = u - row * tile_slots;
          *(lds_u32x4*)(XB0 + row * pitch + rem * 16) = v;
        } else {
          const Slot t = slot_of(u, chunk0);
          if (t.any && t.fast) {
            const unsigned h[5] = {v.x & 0xffffu, v.x >> 16, v.y & 0xffffu, v.y >> 16, v.z & 0xffffu};
            v = finish(h, t);
          }
          *(lds_u32x4*)(XB0 + t.row * pitch + t.rem * 16) = v;
        }
      }
    }
  };

  float total[NQ];
#pragma unroll
  for (int q = 0; q < NQ; ++q) total[q] = 0.f;

  const unsigned stile = (unsigned)(XB0 + tile_rows * pitch);                       // scale tile (SL)
  const unsigned slane = stile + (unsigned)((wave * 16 + r16) * (int)a.G * SB);     // this lane's row of it

  for (int term = 0; term < a.n_terms; ++term) {
    // this wave's 16 rows as a buffer that ends with the tensor; 4-byte aligned base, per-lane row offset
    const unsigned char* wbeg = a.packed[term];
    const unsigned char* wave_rows = wbeg + (e * a.N + n0) * a.Kp;
    const unsigned mis = (unsigned)((uintptr_t)wave_rows & 3);
    const __amdgpu_buffer_rsrc_t wrs = make_rsrc(wave_rows - mis, whole_dwords((wbeg + a.E * a.N * a.Kp) - (wave_rows - mis)));
    const unsigned ro = mis + (unsigned)r16 * (unsigned)a.Kp;
    const unsigned dlt = ro & 3u;            // chunk byte j of this lane's row sits at offset j + dlt of its buffer row
    const unsigned voff_row = ro & ~3u, voff = voff_row + 16u * b;
    const __amdgpu_buffer_rsrc_t srs = make_rsrc((const unsigned char*)a.w_scale[term] + (e * a.N + n0) * a.G * SB, 16 * a.G * SB);
    const int sb = b < 3 ? b : 2;
    const unsigned soff_lane = (unsigned)r16 * (unsigned)a.G * SB + (SDT == BP_F32 ? 8u : 4u) * sb;
    const unsigned rbuf0 = (unsigned)(WB + ((wave * 2) * 16 + r16) * WROW);  // this lane's row in the wave's buffers

    u32x4 wq[2][2] = {};
    unsigned wt[2] = {}, sq[2] = {};
    u32x2 sq2[2] = {};  // (float32 scales)
    auto fetch_pair = [&](int c) {  // chunks c and c + 1 (clamped to the last one)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int cl = c + j < nchunks ? c + j : nchunks - 1;
        const unsigned so = 128u * cl;
        if (ABL == 5) {  // ablation: no weight traffic
          asm volatile("" : "+v"(wq[j][0]), "+v"(wq[j][1]), "+v"(wt[j]));
          continue;
        }
        wq[j][0] = buf_load16(wrs, voff, so);
        wq[j][1] = buf_load16(wrs, voff, so + 64);
        wt[j] = buf_load4(wrs, voff_row, so + 128);
        if (!SL && SDT == BP_F32) {  // k-blocks 0..2 fetch two scales each: groups 5 cl .. 5 cl + 5 (past the rows: zeros)
          sq2[j] = buf_load8(srs, soff_lane, 4u * ((5 * cl) >> gs));
        } else if (!SL) {  // k-blocks 0..2 fetch one dword each = 2 of the 6 scales starting at an even group index
          int gi = ((5 * cl) >> gs) & ~1;
          if (gi > (int)a.G - 6) gi = (int)a.G - 6;
          sq[j] = buf_load4(srs, soff_lane, 2u * gi);
        }
      }
    };

    int next_tile = MULTI ? 0 : nchunks + 2;  // chunk at which the next tile is staged
    int tile_c0 = 0;                            // first chunk of the tile in LDS
    if (MULTI || term == 0) stage_load(0);      // a tile that holds all of K is staged once, for all terms
    fetch_pair(0);
    if (SL) {  // behind the loads above, so that their latencies overlap with the copy's
      const int64_t wg_row0 = (int64_t)blockIdx.x * (WAVES * 16);
      const int64_t wg_rows = a.N - wg_row0 < WAVES * 16 ? a.N - wg_row0 : WAVES * 16;
      const unsigned char* src = (const unsigned char*)a.w_scale[term] + (e * a.N + wg_row0) * a.G * SB;
      const int units16 = (int)(wg_rows * a.G * SB / 16);
      if (term > 0) __syncthreads();  // the previous term's scales are no longer read
      for (int u = threadIdx.x; u < units16; u += THREADS) *(lds_u32x4*)(stile + 16 * u) = *(const u32x4*)(src + 16 * (int64_t)u);
      __syncthreads();
    }
    if (!MULTI && term == 0) {
      __syncthreads();  // (the table is built)
      stage_store(0);
      __syncthreads();
    }

    for (int c = 0; c < nchunks; ++c) {
      if ((c & 1) == 0) {
        // Transpose through the wave's LDS buffers: row r16 of buffer j holds the aligned 128 bytes of chunk
        // c + j and the dword after them. LDS operations of one wave execute in order; the fence only pins
        // the compiler's ordering.
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const unsigned rbj = rbuf0 + j * 16 * WROW;
          *(lds_u32x4*)(rbj + 16 * b) = wq[j][0];
          *(lds_u32x4*)(rbj + 64 + 16 * b) = wq[j][1];
          *(lds_u32*)(rbj + 128) = wt[j];
          if (!SL && SDT == BP_F32) *(lds_u32x2*)(rbj + 136 + 8 * sb) = sq2[j];
          else if (!SL) *(lds_u32*)(rbj + 132 + 4 * sb) = sq[j];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        fetch_pair(c + 2);
      }
      {
        if (MULTI && c == next_tile) {  // uniform for the workgroup
          __syncthreads();  // every wave is done reading the previous tile (and, first time, the table is built)
          stage_store(c);
          __syncthreads();
          tile_c0 = c;
          next_tile += CPT;
          if (next_tile < nchunks) stage_load(next_tile);
        }
        const unsigned rb = rbuf0 + (c & 1) * 16 * WROW;
        const int groups_left = ((int)a.G << gs) - 5 * c;  // 128-wide work groups left in the row
        const int ng = groups_left < 5 ? groups_left : 5;
        int gi = ((5 * c) >> gs) & ~1;
        if (gi > (int)a.G - 6) gi = (int)a.G - 6;
        const int sshift = -gi;  // scale s of the row sits at position s - gi among the 6 loaded (!SL)
        const unsigned xoff = (unsigned)((c - tile_c0) * T1_XCHUNK);
        if (ABL == 1) {  // ablation (timing experiments only): memory traffic without decode and MFMA
#pragma unroll
          for (int g = 0; g < 5; ++g) total[0] += __uint_as_float((*(const lds_u32*)(rb + 24 * g + 4 * b)) & 0x3fffffu);
          continue;
        }
#pragma unroll
        for (int g = 0; g < 5; ++g) {
          if (g < ng) {
            unsigned half;  // the group's scale (bits as stored)
            const int sidx = (5 * c + g) >> gs;  // the 128-wide group's scale (group 256: two of them share one)
            if (SDT == BP_F32) half = SL ? *(const lds_u32*)(slane + 4 * sidx) : *(const lds_u32*)(rb + 136 + 4 * (sidx - ((5 * c) >> gs)));
            else if (SL) half = *(const __attribute__((address_space(3))) uint16_t*)(slane + 2 * sidx);
            else half = *(const __attribute__((address_space(3))) uint16_t*)(rb + 132 + 2 * (sshift + sidx));
            // the 7 bytes of this lane's k-block for group g, read back from the transpose buffer
            const unsigned o = dlt + FB[g] + 7 * b;
            const unsigned d0 = *(const lds_u32*)(rb + (o & ~3u));
            const unsigned d1 = *(const lds_u32*)(rb + (o & ~3u) + 4);
            const unsigned d2 = *(const lds_u32*)(rb + (o & ~3u) + 8);
            const u32x2 wg = {__builtin_amdgcn_alignbyte(d1, d0, o & 3u), __builtin_amdgcn_alignbyte(d2, d1, o & 3u)};
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
            // two-stage pipeline over the 7 MFMA slots: the LDS reads of slot m+1 are issued before the
            // MFMA of slot m; the scheduling barriers keep the compiler from hoisting all 35 slots at once
            u32x4 xa[2];
            u32x2 we[2];
            auto issue = [&](int m, int buf) {
              if (ABL == 4) xa[buf] = u32x4{xaddr, xoff, xaddr, xoff};  // ablation: no activation reads
              else xa[buf] = *(const lds_u32x4*)(xaddr + xoff + 16 * (28 * g + m));
              const unsigned src = m < 4 ? wg.x : wg.y;
              if (ABL == 3) we[buf] = u32x2{(__builtin_amdgcn_ubfe(src, 8 * (m & 3), 8) << 7) | lane_off, src};  // ablation: no table reads
              else we[buf] = *(const lds_u32x2*)((__builtin_amdgcn_ubfe(src, 8 * (m & 3), 8) << 7) | lane_off);
            };
            issue(0, 0);
#pragma unroll
            for (int m = 0; m < 7; ++m) {
              const int cur = m & 1;
              if (m + 1 < 7) issue(m + 1, cur ^ 1);
              // operand dword d = digits 2d (low half) and 2d+1 (high half): entry byte i -> high byte of bf16 i
              const u32x2 en = we[cur];
              const u32x4 d = {__builtin_amdgcn_perm(en.y, en.x, 0x010c000cu), __builtin_amdgcn_perm(en.y, en.x, 0x030c020cu),
                               __builtin_amdgcn_perm(en.y, en.x, 0x0c0c040cu), 0u};
              if (ABL == 2) {  // ablation: everything but the MFMA
                acc[0] += __uint_as_float((d.x ^ d.y ^ d.z ^ xa[cur].x) & 0x3fffffu);
              } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xa[cur]), __builtin_bit_cast(bf16x8, d), acc, 0, 0, 0);
              }
              __builtin_amdgcn_sched_barrier(0);
            }
            // weights were decoded as +-0.5: the factor 2 goes into the scale (exact)
            const float sc = 2.0f * (SDT == BP_F32 ? __uint_as_float(half) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)half) : __uint_as_float(half << 16));
#pragma unroll
            for (int q = 0; q < NQ; ++q) total[q] += acc[q] * sc;
          }
        }
      }
    }
  }
  // ---- epilogue: lane holds tokens 4b + q of output row n0 + r16 (NQ = 1: only token 0 is kept)
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int t = 4 * b + q;
    if (t < ntok && wave_live) {
      float* o = a.out + (tok0 + t) * a.N + n0 + r16;
      *o += x_i8 ? total[q] * a.x_scale[tok0 + t] : total[q];
    }
  }
}

template <int SDT, int WAVES, int NQ, int SL, int MULTI, int ABL = 0>
int launch_tq1_k(const GemmArgs& a, hipStream_t s, const char* name, int64_t cpt, int64_t tokens, size_t lds) {
  const int64_t rows_per_wg = (int64_t)WAVES * 16;
  const dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), (unsigned)a.E, (unsigned)((a.max_rows + 15) / 16));
  if (const int rc = raise_lds_limit<k_mfma_tq1<SDT, WAVES, NQ, SL, MULTI, ABL>>(T1_LDS_MAX)) return rc;
  note_kernel(name);
  hipLaunchKernelGGL((k_mfma_tq1<SDT, WAVES, NQ, SL, MULTI, ABL>), grid, dim3(WAVES * 64), lds, s, a, (int)cpt, (int)tokens);
  return check_launch(name);
}

template <int SDT, int WAVES, int NQ, int SL, int ABL = 0>
int launch_tq1(const GemmArgs& a, hipStream_t s, const char* name) {
  const int64_t rows_per_wg = (int64_t)WAVES * 16;
  // (grid and launch: launch_tq1_k)
  const int64_t tokens = a.max_rows < 16 ? a.max_rows : 16;
  const int64_t nchunks = (a.K + 639) / 640;
  int64_t cpt = (T1_X_BUDGET / tokens - 16) / T1_XCHUNK;
  if (cpt > nchunks) cpt = nchunks;
  if (cpt < 1) return fail(BP_ERR_UNSUPPORTED, "activation tile does not fit");
  const size_t lds = t1_x_base<WAVES, SL, SDT>() + (size_t)tokens * (cpt * T1_XCHUNK + 16) + (SL ? (size_t)rows_per_wg * a.G * (SDT == BP_F32 ? 4 : 2) : 0);
  if (lds > (size_t)T1_LDS_MAX) return BP_ERR_UNSUPPORTED;  // the caller tries the next variant
  if (cpt < nchunks) return launch_tq1_k<SDT, WAVES, NQ, SL, 1, ABL>(a, s, name, cpt, tokens, lds);
  return launch_tq1_k<SDT, WAVES, NQ, SL, 0, ABL>(a, s, name, cpt, tokens, lds);
}

template <int WAVES, int NQ>
int launch_tq1_v(const GemmArgs& a, hipStream_t s, const char* name_sl, const char* name_gl) {
  // scales through the LDS tile when they are 16-byte aligned and everything fits, else per-chunk loads
  bool aligned = true;
  for (int t = 0; t < a.n_terms; ++t) aligned = aligned && ((uintptr_t)a.w_scale[t] & 15) == 0;
  if (aligned) {
    const int rc = a.scale_dtype == BP_F16 ? launch_tq1<BP_F16, WAVES, NQ, 1>(a, s, name_sl)
                   : a.scale_dtype == BP_BF16 ? launch_tq1<BP_BF16, WAVES, NQ, 1>(a, s, name_sl) : launch_tq1<BP_F32, WAVES, NQ, 1>(a, s, name_sl);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  const int rc = a.scale_dtype == BP_F16 ? launch_tq1<BP_F16, WAVES, NQ, 0>(a, s, name_gl)
                 : a.scale_dtype == BP_BF16 ? launch_tq1<BP_BF16, WAVES, NQ, 0>(a, s, name_gl) : launch_tq1<BP_F32, WAVES, NQ, 0>(a, s, name_gl);
  if (rc == BP_ERR_UNSUPPORTED) return fail(BP_ERR_UNSUPPORTED, "TQ1 tile does not fit in LDS");
  return rc;
}

}  // namespace

int launch_mfma_tq1(const GemmArgs& a, hipStream_t s, int waves) {
#ifdef BP_DEV_ABLATIONS  // timing ablations (results are wrong): development builds only
  if (const char* t = getenv("BP_TUNE_ABL")) {
    if (atoi(t) == 1) return launch_tq1<BP_F16, 16, 1, 1, 1>(a, s, "abl1_tq1");
    if (atoi(t) == 2) return launch_tq1<BP_F16, 16, 1, 1, 2>(a, s, "abl2_tq1");
    if (atoi(t) == 3) return launch_tq1<BP_F16, 16, 1, 1, 3>(a, s, "abl3_tq1");
    if (atoi(t) == 4) return launch_tq1<BP_F16, 16, 1, 1, 4>(a, s, "abl4_tq1");
    if (atoi(t) == 5) return launch_tq1<BP_F16, 16, 1, 1, 5>(a, s, "abl5_tq1");
  }
#endif
  if (a.max_rows == 1) {  // decode GEMV
    if (tuning().tq1 != 'm') return launch_tq1_gemv(a, s, waves);  // (development: "mfma" keeps the single-token MFMA variant)
    // one token, only its sums are scaled and kept
    if (waves == 16) return launch_tq1_v<16, 1>(a, s, "mfma_tq1_bf16_t1_w16", "mfma_tq1_bf16_t1_w16_gs");
    return launch_tq1_v<8, 1>(a, s, "mfma_tq1_bf16_t1_w8", "mfma_tq1_bf16_t1_w8_gs");
  }
  if (a.max_rows <= 64) {  // small decode batches: the fp8 x fp4 kernel with one operand tile per token
    if (a.stage && tuning().tq1 == 0 && tuning().tq2g != 'b' && tq1_rows_on_tiles(a.max_rows, a.E, a.T, a.N)) {  // (dense batches of 7 - 8 rows with a workspace)
      const int rc = launch_gemm_tq2f(a, s);
      if (rc != BP_ERR_UNSUPPORTED) return rc;
    }
    if (tuning().tq1 != 'm' && tuning().tq1 != 'l') {  // (development: "mfma" / "lut" keep the kernels below)
      const int rc = launch_tq1_gemv_fp4(a, s);
      if (rc != BP_ERR_UNSUPPORTED) return rc;
    }
  }
  {  // more rows per expert: token tiles of 32 on the fp8 x fp4 matrix instruction - unless the launch would be a few
    // dozen workgroups (one dense linear on a decode batch: 512 rows x 32 tokens each): the 16-token kernel below makes
    // eight times as many and takes half the time there
    const bool few = a.E == 1 && ((a.N + 511) / 512) * ((a.max_rows + 31) / 32) < 64 && a.max_rows <= 128;
    if (tuning().tq1 != 'm' && !few) {  // (development: "mfma" keeps the 16-token kernel below)
      const int rc = launch_gemm_tq1(a, s);
      if (rc != BP_ERR_UNSUPPORTED) return rc;
    }
  }
  if (waves == 16) return launch_tq1_v<16, 4>(a, s, "mfma_tq1_bf16_m1_w16", "mfma_tq1_bf16_m1_w16_gs");
  return launch_tq1_v<8, 4>(a, s, "mfma_tq1_bf16_m1_w8", "mfma_tq1_bf16_m1_w8_gs");
}

}  // namespace bp

// TQ2 decode GEMV (one token row per expert) on the block-float matrix instruction v_mfma_f32_16x16x128_f8f6f4:
// weights as fp4, activations as fp8 (E4M3) pieces, the waves of a workgroup split K.
//
// Contract as everywhere (boilerplate/kernels/ternary_cuda.py:58-63): out[n] += sum_g scale[n, g] * sum_{k in g}
// x[k] * trit[n, k], float32 accumulation; a 2-bit code c stands for the trit c - 1 (boilerplate/ternary/pack.py:34-60).
// The code 3, which pack never writes, counts as +2 as in unpack (the reference's CPU kernel,
// boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77, takes only a trit's sign: +1 there).
//
//  * No decode table and no bit spreading: a packed dword d holds 16 codes, and d & 0x33333333 / (d >> 2) & 0x33333333
//    are two dwords of 8 nibbles whose low two bits are a code. As E2M1 the nibbles 0, 1, 2, 3 read 0, 0.5, 1, 1.5 =
//    c / 2: three vector instructions turn 16 codes into a quarter of operand B. The products then carry sum x * c / 2;
//    every accumulator row starts from - sum x / 2 over its group (computed once per workgroup and wave, exactly: the
//    pieces are fp8 values), which leaves sum x * (c - 1) / 2, and the factor 2 rides on the group's inverse prescale.
//  * K order inside a matrix instruction is free as long as both operands agree: a lane multiplies the 16 bytes it
//    loaded (row n = lane % 16 of a 16-row tile, 16-byte quarter kb = lane / 16 of a 64-byte step = 256 weights = two
//    scale groups of 128) where they are, 8 bytes per instruction.
//  * The 16 rows of operand A are (scale group, piece): a wave owns KV_S = 2 steps = 4 scale groups of 128 of every row,
//    an activation is split into three fp8 pieces as in bp_tq1_gemv_fp4.hip (prescaled per group by a power of two that
//    brings the group's largest magnitude into [128, 256); bf16, fp16 and int8 values are exactly p0 + p1 + p2 / 256
//    down to 2^-20 of the group's largest magnitude), row 4 g + p holds piece p of group g and zeros elsewhere. One
//    accumulator tile collects a tile's four group sums of the wave, a lane of the result (rows 4 kb + i of column n)
//    holds the three pieces of group kb of row n: total = scale[n, g] * (C0 + C1 + C2 / 256) / prescale[g].
//  * Wave w keeps its part of operand A (steps 2 w, 2 w + 1 of the token: 4 instructions x 8 registers) in registers
//    for the whole launch - built straight from the activations in global memory, no LDS tile - and walks over the
//    workgroup's row tiles: per tile two 16-byte loads per lane (16 rows x 128 bytes per wave: whole memory lines, the
//    workgroup's waves together a tile's contiguous 16 x Kp bytes), four tiles in flight in a ring of registers.
//  * A round is 8 tiles. The scales of a round (8 x 16 rows x G entries, contiguous) are loaded at the start of the
//    round before, 16 bytes per lane, and parked in LDS at its end (two slots): one barrier per round, no wait for a
//    load that is younger than the ring's. A wave's 16 partial sums of a tile (its four groups of every row) go to LDS
//    and stay there: after a term's last round thread o adds the waves' sums of the workgroup's output o in wave order
//    (same bits every run). What the call adds to is read when the workgroup starts and written once at its end.
//  * Accuracy: the instruction adds its 128 products in an aligned sum that is narrower than float32 when their
//    magnitudes differ widely: rel-L2 1e-7 to 4e-6 against the CPU kernel on normal activations, 1e-4 when a group holds
//    values four decades apart (the TQ1 kernels on the same instruction: 3e-5); int8 activations are exact.
//
// Operand layout of the instruction with A = fp8 (8 VGPRs), B = fp4 (4 VGPRs), as in bp_tq1_gemv_fp4.hip: B lane
// (n, kb), VGPR w, nibble q is paired with A lane (m, kbA = 2 (kb % 2) + w / 2), VGPR 4 (kb / 2) + 2 (w % 2) + q / 4,
// byte q % 4; C lane (n, lg) holds rows 4 lg + i. With B VGPRs = (even codes of dword 0, odd codes of dword 0, even
// codes of dword 1, odd codes of dword 1) of the instruction's 8 bytes, A lane (row, kbA) VGPR v byte b meets the weight
// 128 (v / 4) + 64 (kbA / 2) + 32 h + 16 (kbA % 2) + 8 (v % 2) + 2 b + (v / 2) % 2 of the step (h: the instruction's
// half of the lane's 16 bytes): per half 16 consecutive activations per lane.
#include <type_traits>

#include "bp_mfma.h"

namespace bp {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
template <int V>
using IC = std::integral_constant<int, V>;

constexpr int KV_S = 2;  // steps (64 packed bytes of a row: 256 weights) per wave
constexpr int KV_R = 8;  // tiles per round (a barrier per round)
constexpr int KV_D = 4;  // tiles in flight per wave
constexpr int KV_OPT = 4;  // outputs per thread at most: a workgroup's tiles are at most 16 x its waves
constexpr unsigned KV_PAST = 0x7ffffff0u;  // an offset past every buffer: the load returns zeros and touches no memory
static_assert(KV_R % KV_D == 0, "the ring's slots are static within a round");

__device__ __forceinline__ float kv_quad_sum(float v) {  // over the lanes n, n + 16, n + 32, n + 48, in a fixed order
  const auto h32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(h32[0]) + __uint_as_float(h32[1]);
  const auto h16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(h16[0]) + __uint_as_float(h16[1]);
}

// 16 consecutive activations of row `row` from element k0 (a multiple of 16): the raw bytes (zeros past K), and as floats
struct KvRun { u32x4 q0, q1; };
__device__ __forceinline__ KvRun kv_load_run(const GemmArgs& a, int64_t row, int64_t k0) {
  KvRun r = {u32x4{0u, 0u, 0u, 0u}, u32x4{0u, 0u, 0u, 0u}};
  if (k0 + 16 > a.K) return r;
  if (a.x_dtype == BP_I8) {
    r.q0 = *(const u32x4*)((const int8_t*)a.x + row * a.K + k0);
  } else {
    const u32x4* src = (const u32x4*)((const uint16_t*)a.x + row * a.K + k0);
    r.q0 = src[0];
    r.q1 = src[1];
  }
  return r;
}
__device__ __forceinline__ void kv_widen_run(const GemmArgs& a, const KvRun& r, float (&y)[16]) {
  if (a.x_dtype == BP_I8) {
#pragma unroll
    for (int t = 0; t < 16; ++t) y[t] = (float)(int)(int8_t)((r.q0[t >> 2] >> (8 * (t & 3))) & 0xffu);
    return;
  }
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    const unsigned w = t < 8 ? r.q0[(t & 7) >> 1] : r.q1[(t & 7) >> 1];
    const uint16_t h = (uint16_t)((t & 1) ? w >> 16 : w & 0xffffu);
    y[t] = a.x_dtype == BP_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
  }
}

// NTOK = 2: a pair of token rows per expert (bf16 / int8 activations: two fp8 pieces suffice, as in the small-batch TQ1
// kernels - exact down to 2^-9 of a group's largest magnitude, at most 2^-17 of it dropped below). Row 4 g + 2 t + p of
// operand A is piece p of token t in group g: the same 4 x 8 registers per wave, one accumulator tile per row tile, and
// a lane of the result holds both tokens' pieces of group kb.
template <int SDT, int NTOK = 1>
__global__ __launch_bounds__(1024) void k_tq2_gemv_ks(GemmArgs a, int nw, int tiles_per_wg) {
  static_assert(NTOK == 1 || NTOK == 2 || NTOK == 4, "one token row per expert, a pair, or four");
  // NTOK = 4: the matrix instructions of a step (two of a tile's four) meet only that step's two groups, so with an
  // accumulator tile per step the 16 rows are 2 groups x 4 tokens x 2 pieces: row 8 q + 2 t + p is piece p of token t in
  // the step's group q, and a lane builds its row for both steps (groups q and 2 + q of the wave's four).
  constexpr bool M4 = NTOK == 4;
  constexpr int SB = SDT == BP_F32 ? 4 : 2, NSL = SB / 2;  // bytes per scale; a wave's 16-byte loads of a round's scales
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int n = lane & 15, kb = lane >> 4;
  const int64_t e = blockIdx.y;
  const int64_t tok = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  if (tok >= o1) return;  // (uniform: an expert without a token row)
  const int ntok = o1 - tok < NTOK ? (int)(o1 - tok) : NTOK;
  float xsc[NTOK];
#pragma unroll
  for (int tt = 0; tt < NTOK; ++tt) xsc[tt] = a.x_dtype == BP_I8 && tt < ntok ? a.x_scale[tok + tt] : 1.f;
  const int gs = a.group == 256 ? 1 : 0;
  const int64_t tiles = a.N / 16;
  const int64_t tile0 = (int64_t)blockIdx.x * tiles_per_wg;
  const int64_t tile_end = tile0 + tiles_per_wg < tiles ? tile0 + tiles_per_wg : tiles;
  const int nrounds = (int)((tile_end - tile0 + KV_R - 1) / KV_R);

  // ---- LDS: two slots of a round's scales, then two of a round's partial sums [tile][wave][row]
  const unsigned row_sb = (unsigned)(a.G * SB), tile_sb = 16 * row_sb, slot_bytes = KV_R * tile_sb;
  const unsigned RED = 2 * slot_bytes;  // [tile of the workgroup][wave][token][row]
  // the lane's group of 128 as a column of the result (four tokens: group kb / 2 of the first step, and 2 + kb / 2 of the second)
  const int64_t g128 = 2 * KV_S * (int64_t)wave + (M4 ? kb >> 1 : kb), g128b = g128 + 2;
  const bool g_real = 128 * g128 < a.K, g_realb = M4 && 128 * g128b < a.K;
  const unsigned rd_s = (unsigned)n * row_sb + (unsigned)SB * (unsigned)(g_real ? g128 >> gs : 0);
  const unsigned rd_sb = (unsigned)n * row_sb + (unsigned)SB * (unsigned)(g_realb ? g128b >> gs : 0);
  const unsigned w_lane = (unsigned)n * (unsigned)a.Kp + 16u * (unsigned)kb + 64u * KV_S * (unsigned)wave;
  const unsigned s_off = 16u * (unsigned)(64 * wave + lane), s_step = 1024u * (unsigned)nw;  // (load j of a wave: + j s_step)

  // The lane as a row of operand A: piece p of the wave's group gl (p = 3: unused); its 2 x 16 activations are requested
  // first, the first tiles next, and operand A is built while those are on their way.
  // (several tokens: the lane's token; four: gl is the lane's group of the first step, gl + 2 that of the second)
  const int gl = M4 ? n >> 3 : n >> 2, p = NTOK >= 2 ? n & 1 : n & 3, trow = M4 ? (n >> 1) & 3 : NTOK == 2 ? (n >> 1) & 1 : 0;
  const int64_t kbase = 256 * KV_S * (int64_t)wave + 128 * gl + 64 * (kb >> 1) + 16 * (kb & 1);
  // (an expert with fewer rows: the absent tokens' rows of operand A hold zeros, their sums are not stored)
  const int64_t kx = trow < ntok ? kbase : a.K, kxb = M4 && trow < ntok ? kbase + 256 : a.K;
  const KvRun x_lo = kv_load_run(a, tok + trow, kx), x_hi = kv_load_run(a, tok + trow, kx + 32);
  const KvRun xb_lo = kv_load_run(a, tok + trow, kxb), xb_hi = kv_load_run(a, tok + trow, kxb + 32);  // (four tokens: the second step's group)
  // Thread o of the workgroup owns output o of the workgroup's rows (up to KV_OPT of them: o + a multiple of the
  // workgroup's threads): what the call adds to is read now and written back once, after the last term.
  // (a pair: output o = ((tile * 2 + token) * 16 + row)
  const int n_out = (int)(tile_end - tile0) * 16 * NTOK;
  auto out_at = [&](int o) -> int64_t { return (tok + ((o >> 4) % NTOK)) * a.N + tile0 * 16 + ((o >> 4) / NTOK) * 16 + (o & 15); };
  auto out_live = [&](int o) { return o < n_out && ((o >> 4) % NTOK) < ntok; };
  float total[KV_OPT];
#pragma unroll
  for (int u = 0; u < KV_OPT; ++u) {
    const int o = (int)threadIdx.x + u * nw * 64;
    total[u] = out_live(o) ? a.out[out_at(o)] : 0.f;
  }
  i32x8 A[2 * KV_S];
  float cinit[4], inv2[NTOK], cinitb[4], inv2b[2];  // (b: four tokens, the second step; inv2 / inv2b then hold the lane's two tokens)

  // (the expert's rows and scales of a term as buffers of their own: what lies past them reads as zeros)
  __amdgpu_buffer_rsrc_t wrs = make_rsrc(a.packed[0] + e * a.N * a.Kp, a.N * a.Kp);
  __amdgpu_buffer_rsrc_t srs = make_rsrc((const unsigned char*)a.w_scale[0] + e * a.N * a.G * SB, a.N * a.G * SB);
  u32x4 ring[KV_D][KV_S], sc_next[NSL];
  auto request = [&](int t, auto slot_c) {  // the wave's bytes of the workgroup's tile t
    constexpr int slot = decltype(slot_c)::value;
    const int64_t tile = tile0 + t;
    const unsigned so = tile < tile_end ? (unsigned)tile * 16u * (unsigned)a.Kp : KV_PAST;
#pragma unroll
    for (int s = 0; s < KV_S; ++s) ring[slot][s] = buf_load16(wrs, w_lane, so + (tile < tile_end ? 64u * s : 0u));
  };
  auto request_scales = [&](int r) {  // the wave's 1024-byte pieces of round r's scales
    const int64_t tile = tile0 + (int64_t)KV_R * r;
#pragma unroll
    for (int j = 0; j < NSL; ++j) sc_next[j] = buf_load16(srs, s_off + j * s_step < slot_bytes ? s_off + j * s_step : KV_PAST, r < nrounds ? (unsigned)tile * tile_sb : KV_PAST);
  };
  auto park_scales = [&](int r) {
#pragma unroll
    for (int j = 0; j < NSL; ++j)
      if (s_off + j * s_step < slot_bytes) *(lds_u32x4*)((unsigned)(r & 1) * slot_bytes + s_off + j * s_step) = sc_next[j];
  };
  auto multiply = [&](int r, auto i_c) {  // tile i of round r: multiply, request the tile KV_D further on, scale, park the sums
    constexpr int i = decltype(i_c)::value, slot = i % KV_D;
    const unsigned sat = (unsigned)(r & 1) * slot_bytes + (unsigned)i * tile_sb + rd_s;
    const unsigned raw = SB == 4 ? *(const lds_u32*)sat : (unsigned)*(const lds_u16*)sat;
    const unsigned satb = (unsigned)(r & 1) * slot_bytes + (unsigned)i * tile_sb + rd_sb;
    const unsigned rawb = !M4 ? 0u : SB == 4 ? *(const lds_u32*)satb : (unsigned)*(const lds_u16*)satb;
    f32x4 C = {cinit[0], cinit[1], cinit[2], NTOK >= 2 ? cinit[3] : 0.f};
    f32x4 Cb = {cinitb[0], cinitb[1], cinitb[2], cinitb[3]};  // (four tokens: the second step's accumulator tile)
#pragma unroll
    for (int s = 0; s < KV_S; ++s) {
      const u32x4 W = ring[slot][s];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const unsigned d0 = W[2 * h], d1 = W[2 * h + 1];
        const i32x8 B8 = {(int)(d0 & 0x33333333u), (int)((d0 >> 2) & 0x33333333u), (int)(d1 & 0x33333333u), (int)((d1 >> 2) & 0x33333333u), 0, 0, 0, 0};
        if (M4 && s == 1) Cb = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[2 * s + h], B8, Cb, 0, 4, 0, 0, 0, 0);
        else C = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[2 * s + h], B8, C, 0 /* A: E4M3 */, 4 /* B: E2M1 */, 0, 0, 0, 0);
      }
    }
    request(KV_R * r + i + KV_D, IC<slot>{});
    auto widen = [&](unsigned q) { return SDT == BP_F32 ? __uint_as_float(q) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)q) : __uint_as_float(q << 16); };
    const float sc = widen(raw);
    if constexpr (M4) {  // the lane: group kb / 2 of either step, tokens 2 (kb % 2) and 2 (kb % 2) + 1; the other group's lane is kb ^ 2
      const float scb = widen(rawb);
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        float v = (g_real ? sc * inv2[t2] * (C[2 * t2] + C[2 * t2 + 1]) : 0.f) + (g_realb ? scb * inv2b[t2] * (Cb[2 * t2] + Cb[2 * t2 + 1]) : 0.f);
        const auto h32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(h32[0]) + __uint_as_float(h32[1]);
        const int tt = 2 * (kb & 1) + t2;
        if (kb < 2) *(lds_u32*)(RED + (unsigned)((((KV_R * r + i) * nw + wave) * NTOK + tt) * 64 + 4 * n)) = __float_as_uint(v);
      }
    } else {
#pragma unroll
      for (int tt = 0; tt < NTOK; ++tt) {
        float v = !g_real ? 0.f : NTOK == 2 ? sc * inv2[tt] * (C[2 * tt] + C[2 * tt + 1]) : sc * inv2[0] * (C[0] + C[1] + C[2] * (1.f / 256.f));
        v = kv_quad_sum(v);
        if (kb == 0) *(lds_u32*)(RED + (unsigned)((((KV_R * r + i) * nw + wave) * NTOK + tt) * 64 + 4 * n)) = __float_as_uint(v);
      }
    }
  };

  auto first_requests = [&] {  // a term's first loads: the scales of round 0, the ring's tiles
    request_scales(0);
    request(0, IC<0>{});
    request(1, IC<1>{});
    request(2, IC<2>{});
    request(3, IC<3>{});
  };
  first_requests();

  // ---- the wave's part of operand A, the starting values of an accumulator tile and the lane's inverse prescale
  {
    // the lane's row for the wave's group gidx: its 2 x 16 activations as pieces (word), the sum of the lane's piece over
    // the row's four lanes (hs) and the group's doubled inverse prescale (inv)
    auto build = [&](const KvRun& lo, const KvRun& hi, int gidx, unsigned (&word)[2][4], float& hs, float& inv) {
      float y[2][16];
      kv_widen_run(a, lo, y[0]);
      kv_widen_run(a, hi, y[1]);
      unsigned m = 0;
#pragma unroll
      for (int t = 0; t < 32; ++t) {
        const unsigned v = __float_as_uint(y[t >> 4][t & 15]) & 0x7fffffffu;
        m = m > v ? m : v;
      }
      {  // the group's largest magnitude: the four lanes of a row hold its 128 activations
        unsigned o = (unsigned)__shfl_xor((int)m, 16, 64);
        m = m > o ? m : o;
        o = (unsigned)__shfl_xor((int)m, 32, 64);
        m = m > o ? m : o;
      }
      const bool real = 256 * KV_S * (int64_t)wave + 128 * gidx < a.K;
      int sh = 0;
      bool finite = true;
      if (a.x_dtype != BP_I8) {  // (int8 values fit as they are: prescale 1)
        const int ex = (int)(m >> 23);
        finite = ex != 255;  // a NaN or an infinity among the group's activations
        sh = 134 - ex;
        sh = sh > 120 ? 120 : sh < -120 ? -120 : sh;
      }
      const float pre = __uint_as_float((unsigned)(sh + 127) << 23);
      // twice the inverse prescale (the weights are multiplied as c / 2); NaN for a group with a non-finite activation,
      // so the token's outputs are NaN rather than finite and wrong
      inv = !real ? 0.f : finite ? __uint_as_float((unsigned)(128 - sh) << 23) : __uint_as_float(0x7fc00000u);
      hs = 0.f;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int vv = 0; vv < 4; ++vv) {
          float r[4];
#pragma unroll
          for (int b = 0; b < 4; ++b) r[b] = y[h][8 * (vv & 1) + 2 * b + (vv >> 1)] * pre;
          unsigned mine = 0;
#pragma unroll
          for (int pp = 0; pp < 3; ++pp) {
            const float f = pp == 2 ? 256.f : 1.f;
            int w = __builtin_amdgcn_cvt_pk_fp8_f32(r[0] * f, r[1] * f, 0, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(r[2] * f, r[3] * f, w, true);
            const float f0 = __builtin_amdgcn_cvt_f32_fp8(w, 0), f1 = __builtin_amdgcn_cvt_f32_fp8(w, 1);
            const float f2 = __builtin_amdgcn_cvt_f32_fp8(w, 2), f3 = __builtin_amdgcn_cvt_f32_fp8(w, 3);
            if (pp == p) {
              mine = (unsigned)w;
              hs += (f0 + f1) + (f2 + f3);
            }
            if (pp < 2) { r[0] -= f0; r[1] -= f1; r[2] -= f2; r[3] -= f3; }
          }
          word[h][vv] = mine;
        }
      }
      hs += __shfl_xor(hs, 16, 64);
      hs += __shfl_xor(hs, 32, 64);
    };
    unsigned word[2][4];
    float hs, inv;
    build(x_lo, x_hi, gl, word, hs, inv);
    // (the lane as a column of the result: rows 4 kb + i; one token: row 3 is unused, its sum 0)
#pragma unroll
    for (int i = 0; i < 4; ++i) cinit[i] = -0.5f * __shfl(hs, 4 * kb + i, 64);
    if constexpr (M4) {
      unsigned wordb[2][4];
      float hsb, invb;
      build(xb_lo, xb_hi, gl + 2, wordb, hsb, invb);
#pragma unroll
      for (int i = 0; i < 4; ++i) cinitb[i] = -0.5f * __shfl(hsb, 4 * kb + i, 64);
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        inv2[t2] = __shfl(inv, 4 * kb + 2 * t2, 64);
        inv2b[t2] = __shfl(invb, 4 * kb + 2 * t2, 64);
      }
      inv2[2] = inv2[3] = 0.f;
      // instruction 2 s + h: the step's two groups sit in register halves 0 and 1; the lane's row belongs to half gl
#pragma unroll
      for (int jj = 0; jj < 2 * KV_S; ++jj) {
#pragma unroll
        for (int v = 0; v < 8; ++v) A[jj][v] = (v >> 2) == gl ? (int)((jj >> 1) ? wordb[jj & 1][v & 3] : word[jj & 1][v & 3]) : 0;
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) cinitb[i] = 0.f;
      inv2b[0] = inv2b[1] = 0.f;
#pragma unroll
      for (int tt = 0; tt < NTOK; ++tt) inv2[tt] = __shfl(inv, 4 * kb + 2 * tt, 64);
#pragma unroll
      for (int jj = 0; jj < 2 * KV_S; ++jj) {
#pragma unroll
        for (int v = 0; v < 8; ++v) A[jj][v] = (jj >> 1) == (gl >> 1) && (v >> 2) == (gl & 1) && p < 3 ? (int)word[jj & 1][v & 3] : 0;
      }
    }
  }

  for (int term = 0; term < a.n_terms; ++term) {
    if (term > 0) {
      wrs = make_rsrc(a.packed[term] + e * a.N * a.Kp, a.N * a.Kp);
      srs = make_rsrc((const unsigned char*)a.w_scale[term] + e * a.N * a.G * SB, a.N * a.G * SB);
      first_requests();
    }
    park_scales(0);
    for (int r = 0; r < nrounds; ++r) {
      __syncthreads();  // (round r's scales are parked, round r - 1 is multiplied)
      request_scales(r + 1);
      multiply(r, IC<0>{}); multiply(r, IC<1>{}); multiply(r, IC<2>{}); multiply(r, IC<3>{});
      multiply(r, IC<4>{}); multiply(r, IC<5>{}); multiply(r, IC<6>{}); multiply(r, IC<7>{});
      // (requested at the round's start, older than the loads of the ring: no wait; the slot was read a round ago)
      park_scales(r + 1);
    }
    __syncthreads();
    // the term's sums: thread o adds the waves' partial sums of output o in wave order
#pragma unroll
    for (int u = 0; u < KV_OPT; ++u) {
      const int o = (int)threadIdx.x + u * nw * 64;
      if (o < n_out) {
        const int tl = (o >> 4) / NTOK, tt = (o >> 4) % NTOK;
        float v = 0.f;
        for (int c = 0; c < nw; ++c) v += __uint_as_float(*(const lds_u32*)(RED + (unsigned)((((tl * nw + c) * NTOK + tt) * 16 + (o & 15)) * 4)));
        float xs = xsc[0];  // (the token's activation scale, without indexing the array by a variable)
#pragma unroll
        for (int q = 1; q < NTOK; ++q) xs = tt == q ? xsc[q] : xs;
        total[u] += a.x_dtype == BP_I8 ? v * xs : v;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < KV_OPT; ++u) {
    const int o = (int)threadIdx.x + u * nw * 64;
    if (out_live(o)) a.out[out_at(o)] = total[u];
  }
}

int kv_cus() {  // compute units of the current device (256 if the query fails)
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 256;
  static std::mutex m;
  static int known[64] = {};
  if (dev < 0 || dev >= 64) return 256;
  std::lock_guard<std::mutex> lock(m);
  if (known[dev] == 0) {
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
    known[dev] = cus;
  }
  return known[dev];
}

template <int SDT, int NTOK>
int launch_kv_n(const GemmArgs& a, hipStream_t s, int nw, int64_t per, const dim3& grid, size_t lds) {
  const char* name = NTOK == 4 ? (a.x_dtype == BP_I8 ? "fp4_tq2_i8_m4_ks" : "fp4_tq2_m4_ks") : NTOK == 2 ? (a.x_dtype == BP_I8 ? "fp4_tq2_i8_m2_ks" : "fp4_tq2_m2_ks")
                                : a.x_dtype == BP_I8 ? "fp4_tq2_i8_t1_ks" : "fp4_tq2_t1_ks";
  note_kernel(name);
  if (const int rc = raise_lds_limit<k_tq2_gemv_ks<SDT, NTOK>>(160 * 1024)) return rc;
  hipLaunchKernelGGL((k_tq2_gemv_ks<SDT, NTOK>), grid, dim3((unsigned)nw * 64), lds, s, a, nw, (int)per);
  return check_launch(name);
}
template <int SDT>
int launch_kv(const GemmArgs& a, hipStream_t s, int nw, int64_t per, const dim3& grid, size_t lds, int ntok) {
  if (ntok == 4) return launch_kv_n<SDT, 4>(a, s, nw, per, grid, lds);
  return ntok == 2 ? launch_kv_n<SDT, 2>(a, s, nw, per, grid, lds) : launch_kv_n<SDT, 1>(a, s, nw, per, grid, lds);
}

}  // namespace

// BP_ERR_UNSUPPORTED (no message) where the kernel does not apply: the caller goes on to its other kernels.
int launch_tq2_gemv_fp4(const GemmArgs& a, hipStream_t s) {
  const char force = tuning().tq2v;
  if (force == 'n') return BP_ERR_UNSUPPORTED;
  if (a.fmt != BP_TQ2 || a.max_rows < 1 || a.max_rows > 4 || a.tiles) return BP_ERR_UNSUPPORTED;
  const int ntok = a.max_rows == 3 ? 4 : (int)a.max_rows;  // (three rows: the variant for four)
  if (a.x_dtype != BP_BF16 && a.x_dtype != BP_I8) return BP_ERR_UNSUPPORTED;
  if (a.scale_dtype != BP_F16 && a.scale_dtype != BP_BF16 && a.scale_dtype != BP_F32) return BP_ERR_UNSUPPORTED;
  const int64_t sb = a.scale_dtype == BP_F32 ? 4 : 2;
  if (a.K % 256 != 0 || a.N % 16 != 0 || (a.group != 128 && a.group != 256) || a.G != a.K / a.group || a.Kp != a.K / 4) return BP_ERR_UNSUPPORTED;
  const int64_t nsteps = a.K / 256, nw = (nsteps + KV_S - 1) / KV_S;
  if (nw < 2 || nw > 16) return BP_ERR_UNSUPPORTED;
  if (a.N * a.Kp >= 0x7fffffe0 - 64 * KV_S * 16 || a.N * a.G * sb >= 0x7fffffe0 || a.N * 4 >= 0x7fffffe0) return BP_ERR_UNSUPPORTED;
  if (((uintptr_t)a.x & 15) != 0) return BP_ERR_UNSUPPORTED;
  for (int t = 0; t < a.n_terms; ++t)
    if (((uintptr_t)a.packed[t] & 15) != 0 || ((uintptr_t)a.w_scale[t] & 15) != 0) return BP_ERR_UNSUPPORTED;
  const int64_t slots = 2 * KV_R * 16 * a.G * sb;  // LDS: the scales of two rounds, then 64 bytes per tile and wave
  const int cus = kv_cus();
  const int64_t per_cu = 16 / nw;  // workgroups that a CU holds: 16 waves of up to 128 registers
  const int64_t resident = (int64_t)cus * per_cu;
  const int64_t experts = a.E < a.T ? a.E : a.T, tiles = a.N / 16;
  int64_t wpe = resident / (experts > 0 ? experts : 1);  // workgroups per expert
  wpe = wpe < 1 ? 1 : wpe;
  int64_t per = (tiles + wpe - 1) / wpe;  // tiles per workgroup, in whole rounds
  // (two workgroups per place one after the other when each still gets four rounds: the CUs end more evenly -
  // 128 experts x 128 tiles at K = 7168: 91.9 against 92.8 us; shorter ranges lose more to the set-up than they gain)
  if (per >= 8 * KV_R) per = (per + 1) / 2;
  per = (per + KV_R - 1) / KV_R * KV_R;
  // Measured against k_mfma_tq2 (N x K from 2048 x 1024 to 7168 x 2048 and 512 x 8192, 1 to 256 experts): ahead or
  // level from two row tiles per CU on with bf16 activations (K = 7168: 1.10 x at 128 experts; K = 4096: 1.33 x at 64;
  // K = 2048: 1.28 x at 128), with int8 ones from 16 tiles per CU (below, 14.2 against 15.7 us); behind at K = 1024.
  // (int8 activations with float32 scales: 105 against 101.7 us for k_mfma_tq2 on the 128 x 2048 x 7168 launch)
  if (force != 'k' && a.x_dtype == BP_I8 && a.scale_dtype == BP_F32) return BP_ERR_UNSUPPORTED;
  if (force != 'k' && (a.K < 2048 || experts * tiles < (a.x_dtype == BP_I8 ? 16 : 2) * (int64_t)cus)) return BP_ERR_UNSUPPORTED;
  // (a thread owns up to KV_OPT outputs; the partial sums of a workgroup's tiles stay in LDS until the term's end)
  const int64_t lds_cap = 160 * 1024 / per_cu;
  // (a thread owns up to KV_OPT outputs; a pair has two per row)
  int64_t per_max = 16 * nw / ntok < (lds_cap - slots) / (nw * 64 * ntok) ? 16 * nw / ntok : (lds_cap - slots) / (nw * 64 * ntok);
  per_max = per_max / KV_R * KV_R;
  if (per_max < 2 * KV_R) return BP_ERR_UNSUPPORTED;
  // (ranges too long for a workgroup's LDS: twice, three times ... as many workgroups per expert, so that the launch
  // stays whole rounds of the resident workgroups - 96 tiles per expert at four rows as 4 x 24, not 3 x 32)
  for (int64_t k = 2; per > per_max; ++k) per = ((tiles + k * wpe - 1) / (k * wpe) + KV_R - 1) / KV_R * KV_R;
  const size_t lds = (size_t)(slots + per * nw * 64 * ntok);
  const dim3 grid((unsigned)((tiles + per - 1) / per), (unsigned)a.E, 1u);
  if (a.E > 65535) return BP_ERR_UNSUPPORTED;
  if (a.scale_dtype == BP_F32) return launch_kv<BP_F32>(a, s, (int)nw, per, grid, lds, ntok);
  return a.scale_dtype == BP_F16 ? launch_kv<BP_F16>(a, s, (int)nw, per, grid, lds, ntok) : launch_kv<BP_BF16>(a, s, (int)nw, per, grid, lds, ntok);
}

}  // namespace bp

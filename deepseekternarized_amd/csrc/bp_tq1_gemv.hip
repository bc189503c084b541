// TQ1 single-token GEMV (decode, one token row per expert) without matrix instructions.
//
// With one token, a 16-token MFMA tile is 1/16 used and the kernel that feeds it is bound by its LDS
// reads (a table entry and an activation operand per packed byte). Here the activations are folded into
// the tables instead: for every byte position the workgroup precomputes, once, the partial dot products of
// that byte's 5 activations with every possible digit pattern, split in two so the tables stay small:
//
//     byte v = r + 9 q,   r = d0 + 3 d1 (9 patterns),   q = d2 + 3 d3 + 9 d4 (27 patterns)
//     T9[r]  = (d0 - 1) x0 + (d1 - 1) x1          T27[q] = (d2 - 1) x2 + (d3 - 1) x3 + (d4 - 1) x4
//
// so a packed byte costs two 4-byte LDS reads and two float adds per output row, whatever its digits.
// q = (v * 57) >> 9 is exact for v < 256; bytes >= 243 do not occur in packed tensors (pack writes
// digits 0..2 only) - the general kernel treats them as zeros, this one reads the tables out of pattern.
//
// Work split as in the MFMA kernel of this format: a wave owns 16 output rows; 640 trits = 128 bytes = 5
// scale groups form a chunk; group g of a chunk is given 28 byte slots, lane (r16 = lane % 16, b = lane /
// 16) taking bytes FB[g] + 7 b + m, m = 0..6, of row r16. A slot's table is built from the activations
// of its byte with the digits of neighbouring groups (or past K, or past the group's last byte) zeroed,
// so every lane runs the same 7 lookups per group and the group's scale multiplies the lane's partial
// sum; the four b-lanes of a row are added once, at the end.
//
// Packed bytes reach the lanes as in the MFMA kernel: aligned 16-byte buffer loads (two chunks back to
// back, reads past the tensor return zeros), transposed through a per-wave LDS buffer.
#include "bp_mfma.h"

namespace bp {
namespace {

struct __attribute__((packed, aligned(2))) Packed16 { u32x4 v; };
typedef __attribute__((address_space(3))) float lds_f32;

constexpr int G1_SLOTS = 140;                     // byte slots per chunk: 5 groups x 28
constexpr int G1_SLOT_BYTES = 44 * 4;             // T9 (9 floats) then T27 (27 floats), padded to 44 banks (see the table tile)
constexpr int G1_CHUNK_BYTES = G1_SLOTS * G1_SLOT_BYTES;
// Row pitch of the transpose buffer, a multiple of 16: 136 data bytes (the aligned 128 of the chunk and the 8
// after them, so that every byte a slot can name - up to chunk byte 129 at a row misalignment of 3 - is a
// byte of the tensor, or the zero a buffer load returns past it, and never stale LDS), + 12 of scales if !SL.
template <int SL>
constexpr int g1_wrow() { return SL ? 144 : 160; }
constexpr int G1_LDS_MAX = 160 * 1024;

__device__ __forceinline__ unsigned g1_load4(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned wave_off) {
  return (unsigned)__builtin_amdgcn_raw_buffer_load_b32(r, (int)lane_off, (int)wave_off, 0);
}
__device__ __forceinline__ u32x2 g1_load8(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned wave_off) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)lane_off, (int)wave_off, 0));
}

// SL: scales through an LDS tile (copied once per workgroup and term) instead of per-chunk loads.
// MULTI: the tables cover only part of K and are rebuilt inside the chunk loop.
template <int SDT, int WAVES, int SL, int MULTI>
__global__ __launch_bounds__(WAVES * 64, 4) void k_tq1_gemv(GemmArgs a, int CPT /* chunks per table tile */) {
  constexpr int THREADS = WAVES * 64;
  constexpr int WROW = g1_wrow<SL>();
  constexpr int TB = WAVES * 16 * WROW;  // tables start after the wave buffers
  constexpr int XU = 2;                  // table slots built per thread (launcher keeps CPT * 140 <= XU * THREADS)
  constexpr int FB[5] = {0, 25, 51, 76, 102};
  constexpr int SB = SDT == BP_F32 ? 4 : 2;  // bytes per scale (float32 scales: scale tile variant only)
  static_assert(SL || SDT != BP_F32, "float32 scales are read through the LDS tile");

  // the wave index through readfirstlane: everything derived from it stays in scalar registers
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, b = lane >> 4;
  const int64_t e = blockIdx.y;
  const int64_t o0 = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  if (o0 >= o1) return;  // uniform for the workgroup; only the expert's first token row is used (max_rows == 1)
  const int64_t tok = o0;
  int64_t n0 = ((int64_t)blockIdx.x * WAVES + wave) * 16;
  const bool wave_live = n0 < a.N;
  if (!wave_live) n0 = 0;  // keeps addresses valid; the wave still takes part in staging and barriers

  const int nchunks = (int)((a.K + 639) / 640);  // 128-byte chunks per row (the last may be partial)
  const int gs = a.group == 256 ? 1 : 0;         // scale groups of 256: two 128-wide work groups share a scale
  const int tile_slots = CPT * G1_SLOTS;
  // ---- table tile: the table of slot (cl, g, 7 b + m) sits at TB + ((cl * 5 + g) * 28 + 4 m + b) * 176.
  // The LDS has 32 banks and serves a wave's 4-byte reads half a wave at a time (measured): lane groups b = 0, 1
  // meet in one pass, b = 2, 3 in the other. Their tables lie one slot = 44 banks = 12 (mod 32) apart, so the T9
  // entries (9 banks) of the two groups of a pass never share a bank; with the tables 7 slots of 36 banks apart
  // they did for most entries, and half of the kernel's LDS cycles were bank conflicts. (Two T27 tables cannot
  // be disjoint in 32 banks.) The thread that builds a table is the one whose index equals the table's
  // position, so a wave's 16-byte stores stay an odd multiple of 4 banks apart (conflict-free).
  float xstage[XU][5];  // the slot's 5 activations, masked (any activation dtype; int8 values are exact in float)
  auto stage_load = [&](int chunk0) {  // global -> registers: the tile that starts at chunk `chunk0`
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      const int u = threadIdx.x + i * THREADS;
#pragma unroll
      for (int d = 0; d < 5; ++d) xstage[i][d] = 0.f;
      if (u < tile_slots) {
        const int cl = u / G1_SLOTS, sg = u - cl * G1_SLOTS;
        const int g = sg / 28, pos = sg - g * 28;                  // position 4 m + b within the group's tables
        const int sl = 7 * (pos & 3) + (pos >> 2);                 // sl = 7 b + m: byte FB[g] + sl of the chunk
        const int j = (g == 0 ? 0 : g == 1 ? 25 : g == 2 ? 51 : g == 3 ? 76 : 102) + sl;
        const int64_t k0 = 640 * (int64_t)(chunk0 + cl) + 5 * j;  // first activation of the byte
        int lo = 128 * g - 5 * j, hi = lo + 128;                   // digits lo <= d < hi belong to group g
        if (a.K - k0 < hi) hi = (int)(a.K - k0);                   // ... and lie inside K
        const int64_t at = tok * a.K + k0;
        if ((a.x_dtype == BP_BF16 || a.x_dtype == BP_F16) && hi > 0 && lo < 5 && k0 + 8 <= a.K) {
          // 16-bit activations away from the row's end: one 16-byte load instead of five 2-byte ones
          const u32x4 q = ((const Packed16*)((const uint16_t*)a.x + at))->v;
          const unsigned h[5] = {q.x & 0xffffu, q.x >> 16, q.y & 0xffffu, q.y >> 16, q.z & 0xffffu};
#pragma unroll
          for (int d = 0; d < 5; ++d)
            if (d >= lo && d < hi) xstage[i][d] = a.x_dtype == BP_BF16 ? bf16_bits_to_f32((uint16_t)h[d]) : f16_bits_to_f32((uint16_t)h[d]);
          continue;
        }
#pragma unroll
        for (int d = 0; d < 5; ++d) {
          if (d >= lo && d < hi) {
            float v;
            if (a.x_dtype == BP_BF16) v = bf16_bits_to_f32(((const uint16_t*)a.x)[at + d]);
            else if (a.x_dtype == BP_F16) v = f16_bits_to_f32(((const uint16_t*)a.x)[at + d]);
            else if (a.x_dtype == BP_F32) v = ((const float*)a.x)[at + d];
            else v = (float)((const int8_t*)a.x)[at + d];
            xstage[i][d] = v;
          }
        }
      }
    }
  };
  auto stage_store = [&]() {  // registers -> the 36 partial sums of every slot
#pragma unroll
    for (int i = 0; i < XU; ++i) {
      const int u = threadIdx.x + i * THREADS;
      if (u < tile_slots) {
        const float x0 = xstage[i][0], x1 = xstage[i][1], x2 = xstage[i][2], x3 = xstage[i][3], x4 = xstage[i][4];
        // entry e of the slot: e < 9 -> T9[e], else T27[e - 9]; written four at a time
        auto entry = [&](int en) -> unsigned {
          if (en < 9) return __float_as_uint((float)(en % 3 - 1) * x0 + (float)(en / 3 - 1) * x1);
          const int q = en - 9;
          return __float_as_uint((float)(q % 3 - 1) * x2 + (float)(q / 3 % 3 - 1) * x3 + (float)(q / 9 - 1) * x4);
        };
        const unsigned dst = (unsigned)(TB + u * G1_SLOT_BYTES);  // (the 32 bytes of padding stay unwritten)
#pragma unroll
        for (int w = 0; w < 9; ++w) {
          *(lds_u32x4*)(dst + 16 * w) = u32x4{entry(4 * w), entry(4 * w + 1), entry(4 * w + 2), entry(4 * w + 3)};
          __builtin_amdgcn_sched_barrier(0);  // one store's worth of values live at a time
        }
      }
    }
  };

  float total = 0.f;
  const unsigned stile = (unsigned)(TB + CPT * G1_CHUNK_BYTES);                     // scale tile (SL)
  const unsigned slane = stile + (unsigned)((wave * 16 + r16) * (int)a.G * SB);     // this lane's row of it
  const unsigned rb = (unsigned)((wave * 16 + r16) * WROW);                         // this lane's row in the wave's buffer

  for (int term = 0; term < a.n_terms; ++term) {
    // this wave's 16 rows as a buffer that ends with the tensor; 4-byte aligned base, per-lane row offset
    const unsigned char* wbeg = a.packed[term];
    const unsigned char* wave_rows = wbeg + (e * a.N + n0) * a.Kp;
    const unsigned mis = (unsigned)((uintptr_t)wave_rows & 3);
    const __amdgpu_buffer_rsrc_t wrs = make_rsrc(wave_rows - mis, whole_dwords((wbeg + a.E * a.N * a.Kp) - (wave_rows - mis)));
    const unsigned ro = mis + (unsigned)r16 * (unsigned)a.Kp;
    const unsigned dlt = ro & 3u;            // chunk byte j of this lane's row sits at offset j + dlt of its buffer row
    const unsigned voff_row = ro & ~3u, voff = voff_row + 16u * b;
    const __amdgpu_buffer_rsrc_t srs = make_rsrc((const unsigned char*)a.w_scale[term] + (e * a.N + n0) * a.G * 2, 16 * a.G * 2);
    const int sb = b < 3 ? b : 2;
    const unsigned soff_lane = (unsigned)r16 * (unsigned)a.G * 2u + 4u * sb;

    u32x4 wq[2][2];
    u32x2 wt[2];
    unsigned sq[2] = {};
    auto fetch_pair = [&](int c) {  // chunks c and c + 1 (clamped to the last one)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int cl = c + j < nchunks ? c + j : nchunks - 1;
        const unsigned so = 128u * cl;
        wq[j][0] = buf_load16(wrs, voff, so);
        wq[j][1] = buf_load16(wrs, voff, so + 64);
        wt[j] = g1_load8(wrs, voff_row, so + 128);
        if (!SL) {  // k-blocks 0..2 fetch one dword each = 2 of the 6 scales starting at an even group index
          int gi = ((5 * cl) >> gs) & ~1;
          if (gi > (int)a.G - 6) gi = (int)a.G - 6;
          sq[j] = g1_load4(srs, soff_lane, 2u * gi);
        }
      }
    };

    int next_tile = MULTI ? 0 : nchunks + 2;  // chunk at which the next tile is built
    int tile_c0 = 0;                            // first chunk of the tile in LDS
    if (MULTI || term == 0) stage_load(0);      // tables that cover all of K are built once, for all terms
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
      stage_store();
      __syncthreads();
    }

    for (int c = 0; c < nchunks; ++c) {
      // Transpose through the wave's LDS buffer: row r16 holds the aligned 128 bytes of the chunk and the
      // dword after them. LDS operations of one wave execute in order; the fences only pin the compiler's
      // ordering. Even chunks come from the first half of the register pair, odd ones from the second,
      // after which the pair is refilled with the next two chunks.
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if ((c & 1) == 0) {
        *(lds_u32x4*)(rb + 16 * b) = wq[0][0];
        *(lds_u32x4*)(rb + 64 + 16 * b) = wq[0][1];
        *(lds_u32x2*)(rb + 128) = wt[0];
        if (!SL) *(lds_u32*)(rb + 136 + 4 * sb) = sq[0];
      } else {
        *(lds_u32x4*)(rb + 16 * b) = wq[1][0];
        *(lds_u32x4*)(rb + 64 + 16 * b) = wq[1][1];
        *(lds_u32x2*)(rb + 128) = wt[1];
        if (!SL) *(lds_u32*)(rb + 136 + 4 * sb) = sq[1];
        fetch_pair(c + 1);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (MULTI && c == next_tile) {  // uniform for the workgroup
        __syncthreads();  // every wave is done reading the previous tables
        stage_store();
        __syncthreads();
        tile_c0 = c;
        next_tile += CPT;
        if (next_tile < nchunks) stage_load(next_tile);
      }
      const int groups_left = ((int)a.G << gs) - 5 * c;  // 128-wide work groups left in the row
      const int ng = groups_left < 5 ? groups_left : 5;
      int gi = ((5 * c) >> gs) & ~1;
      if (gi > (int)a.G - 6) gi = (int)a.G - 6;
      const int sshift = -gi;  // scale s of the row sits at position s - gi among the 6 loaded (!SL)
      // this lane's first table of the chunk; the slot within the chunk is an instruction offset
      unsigned tbl = (unsigned)(TB + (c - tile_c0) * G1_CHUNK_BYTES + G1_SLOT_BYTES * b);
      asm volatile("" : "+v"(tbl));  // one register; the rest of every table address is q, r and an instruction offset
#pragma unroll
      for (int g = 0; g < 5; ++g) {
        if (g < ng) {
          unsigned half;  // the group's scale (bits as stored)
          const int sidx = (5 * c + g) >> gs;  // the 128-wide group's scale (group 256: two of them share one)
          if (SDT == BP_F32) half = *(const lds_u32*)(slane + 4 * sidx);
          else if (SL) half = *(const __attribute__((address_space(3))) uint16_t*)(slane + 2 * sidx);
          else half = *(const __attribute__((address_space(3))) uint16_t*)(rb + 136 + 2 * (sshift + sidx));
          // the 7 bytes of this lane's slots for group g, read back from the transpose buffer
          const unsigned o = dlt + FB[g] + 7 * b;
          const unsigned d0 = *(const lds_u32*)(rb + (o & ~3u));
          const unsigned d1 = *(const lds_u32*)(rb + (o & ~3u) + 4);
          const unsigned d2 = *(const lds_u32*)(rb + (o & ~3u) + 8);
          const u32x2 wg = {__builtin_amdgcn_alignbyte(d1, d0, o & 3u), __builtin_amdgcn_alignbyte(d2, d1, o & 3u)};
          // all 14 addresses, then all 14 reads, then the sums: the reads overlap instead of being waited for one by one
          unsigned a9[7], a27[7];
#pragma unroll
          for (int m = 0; m < 7; ++m) {
            const unsigned v = __builtin_amdgcn_ubfe(m < 4 ? wg.x : wg.y, 8 * (m & 3), 8);
            const unsigned q = __umul24(v, 57u) >> 9;                                      // v / 9
            a27[m] = __umul24(q, 4u) + tbl;                                                 // T27[q]
            a9[m] = (unsigned)(__mul24((int)q, -36) + (int)(__umul24(v, 4u) + tbl));        // T9[v - 9 q]
          }
          float t9[7], t27[7];
#pragma unroll
          for (int m = 0; m < 7; ++m) {
            t9[m] = *(const lds_f32*)(a9[m] + (28 * g + 4 * m) * G1_SLOT_BYTES);
            t27[m] = *(const lds_f32*)(a27[m] + (28 * g + 4 * m) * G1_SLOT_BYTES + 36);
          }
          float acc9 = t9[0], acc27 = t27[0];
#pragma unroll
          for (int m = 1; m < 7; ++m) { acc9 += t9[m]; acc27 += t27[m]; }
          const float sc = SDT == BP_F32 ? __uint_as_float(half) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)half) : __uint_as_float(half << 16);
          total += (acc9 + acc27) * sc;
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  }
  // ---- epilogue: the four b-lanes of a row hold its partial sums
  total += __shfl_xor(total, 16);
  total += __shfl_xor(total, 32);
  if (b == 0 && wave_live) {
    float* o = a.out + tok * a.N + n0 + r16;
    *o += a.x_dtype == BP_I8 ? total * a.x_scale[tok] : total;
  }
}

template <int SDT, int WAVES, int SL, int MULTI>
int launch_g1_k(const GemmArgs& a, hipStream_t s, const char* name, int64_t cpt, size_t lds) {
  const int64_t rows_per_wg = (int64_t)WAVES * 16;
  const dim3 grid((unsigned)((a.N + rows_per_wg - 1) / rows_per_wg), (unsigned)a.E, 1u);
  if (const int rc = raise_lds_limit<k_tq1_gemv<SDT, WAVES, SL, MULTI>>(G1_LDS_MAX)) return rc;
  note_kernel(name);
  hipLaunchKernelGGL((k_tq1_gemv<SDT, WAVES, SL, MULTI>), grid, dim3(WAVES * 64), lds, s, a, (int)cpt);
  return check_launch(name);
}

template <int SDT, int WAVES, int SL>
int launch_g1(const GemmArgs& a, hipStream_t s, const char* name) {
  const int64_t rows_per_wg = (int64_t)WAVES * 16;
  const int64_t nchunks = (a.K + 639) / 640;
  const int64_t fixed = rows_per_wg * g1_wrow<SL>() + (SL ? rows_per_wg * a.G * (SDT == BP_F32 ? 4 : 2) : 0);
  int64_t cpt = (G1_LDS_MAX - fixed) / G1_CHUNK_BYTES;
  const int64_t cap = 2 * WAVES * 64 / G1_SLOTS;  // two table slots per thread at most
  if (cpt > cap) cpt = cap;
  if (tuning().cpt >= 1 && tuning().cpt < cpt) cpt = tuning().cpt;  // (development)
  if (cpt > nchunks) cpt = nchunks;
  if (cpt < 1) return BP_ERR_UNSUPPORTED;  // the caller tries the next variant
  const size_t lds = (size_t)(fixed + cpt * G1_CHUNK_BYTES);
  if (cpt < nchunks) return launch_g1_k<SDT, WAVES, SL, 1>(a, s, name, cpt, lds);
  return launch_g1_k<SDT, WAVES, SL, 0>(a, s, name, cpt, lds);
}

template <int WAVES>
int launch_g1_v(const GemmArgs& a, hipStream_t s, const char* name_sl, const char* name_gl) {
  bool aligned = true;
  for (int t = 0; t < a.n_terms; ++t) aligned = aligned && ((uintptr_t)a.w_scale[t] & 15) == 0;
  if (a.scale_dtype == BP_F32)  // float32 scales (what the reference's own wrappers pass): scale tile or nothing
    return aligned ? launch_g1<BP_F32, WAVES, 1>(a, s, name_sl) : BP_ERR_UNSUPPORTED;
  if (aligned) {
    const int rc = a.scale_dtype == BP_F16 ? launch_g1<BP_F16, WAVES, 1>(a, s, name_sl) : launch_g1<BP_BF16, WAVES, 1>(a, s, name_sl);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  const int rc = a.scale_dtype == BP_F16 ? launch_g1<BP_F16, WAVES, 0>(a, s, name_gl) : launch_g1<BP_BF16, WAVES, 0>(a, s, name_gl);
  if (rc == BP_ERR_UNSUPPORTED) return fail(BP_ERR_UNSUPPORTED, "TQ1 GEMV tables do not fit in LDS");
  return rc;
}

}  // namespace

// max_rows == 1 (checked by the caller); any activation dtype
int launch_tq1_gemv(const GemmArgs& a, hipStream_t s, int waves) {
  if (tuning().tq1 != 'l') {  // (development: "lut" keeps the table kernel)
    const int rc = launch_tq1_gemv_fp4(a, s);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  if (waves == 16) return launch_g1_v<16>(a, s, "lut_tq1_t1_w16", "lut_tq1_t1_w16_gs");
  return launch_g1_v<8>(a, s, "lut_tq1_t1_w8", "lut_tq1_t1_w8_gs");
}

}  // namespace bp

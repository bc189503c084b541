// TQ1 grouped GEMM for token tiles of 16 or 32 rows (experts with more than 8 token rows): tokens are the rows of
// operand A of v_mfma_scale_f32_16x16x128_f8f6f4, packed weights stream once per 32 tokens.
//
// Contract as everywhere (boilerplate/kernels/ternary_cuda.py:58-63, boilerplate/kernels/csrc/ternary_cuda_kernel.cu:44-99):
// out[t, n] += x_scale[t] * sum_g scale[n, g] * sum_{k in g} x[t, k] * trit[n, k], float32 accumulation.
//
//  * Weights as fp4 (E2M1 holds -1, 0, +1 exactly) through the byte -> 5 fp4 codes table of bp_tq1_gemv_fp4.hip (one
//    dword per packed byte, one copy per LDS bank: a conflict-free 4-byte read per byte and no unpacking arithmetic).
//    A packed byte fills 8 of the instruction's 128 k-slots (5 digits, 3 zeros); an instruction covers 16 packed bytes.
//  * A lane loads 16 consecutive bytes of its row per 64-byte window, at the row's own byte alignment (rows start at any
//    byte; the kernel is far from the HBM rate, where a misaligned load would cost). Four lane-quarter swaps
//    (v_permlane32_swap / v_permlane16_swap) transpose the 4 x 4 dwords of a row's window between the four lanes that
//    hold them, so that matrix instruction j of
//    a window multiplies the CONSECUTIVE bytes 16 j .. 16 j + 15 of every row and lies in one 128-wide scale group - or
//    in two, for the 4 of the 8 instructions of a 128-byte chunk (640 digits = 5 groups) in which a group ends. Those
//    run twice, on operand B masked to the digits of the first and of the second group (a lane-dependent AND), so every
//    group sum is collected separately and multiplied by its scale exactly as the reference does: 12 instructions per
//    chunk and activation piece.
//  * Activations as two fp8 (E4M3) pieces under a power-of-two block scale that the instruction itself applies: the 20
//    activations behind 4 consecutive packed bytes (= the 32 k-slots one lane of operand B holds) share one E8M0 scale
//    2^(e - 7), e the exponent of the block's largest magnitude; y = x / scale = p0 + p1 with p0 = y rounded to E4M3 and
//    p1 the rounded remainder. bf16 and int8 activations are exactly p0 + p1 down to 2^-9 of the largest magnitude of
//    their block of 20; what is dropped below that is less than 2^-17 of it. Products fp8 x fp4 are exact. A block that
//    holds a NaN or an infinity makes the token's outputs NaN (never a finite wrong value).
//  * A workgroup (8 waves) owns 512 output rows x 32 tokens; a wave 64 rows (4 row tiles) x 32 tokens (2 token tiles):
//    a table read feeds 4 instructions, an operand A read 4 to 8. The activation operands of one window (32 KiB for 32
//    tokens) are converted by the workgroup itself and double-buffered in LDS, one barrier per window; the scales go
//    through LDS as stored, 8 per row and load. The next window's loads are spread over the window's instruction slots:
//    the memory pipeline takes about 64 clocks per wave-wide load, and a wave that cannot issue a load issues nothing.
//
// Operand layout of the instruction (A = fp8, 8 VGPRs; B = fp4, 4 VGPRs; established by probing on gfx950): B lane
// (n = lane % 16, kb = lane / 16), VGPR w, nibble q is paired with A lane (m = lane % 16, 2 (kb % 2) + w / 2), VGPR
// 4 (kb / 2) + 2 (w % 2) + q / 4, byte q % 4; the E8M0 scale of A row m for the 32 slots of B lane kb is byte `opsel`
// of the scale operand in lane (m, kb); C lane (n, lg) holds rows 4 lg + i.
#include <type_traits>

#include "bp_mfma.h"

namespace bp {
namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
template <int V>
using QC = std::integral_constant<int, V>;

constexpr int Q_WAVES = 8;                         // waves per workgroup
constexpr int Q_RT = 4;                            // 16-row tiles per wave
constexpr int Q_THREADS = Q_WAVES * 64;
constexpr int Q_ROWS = Q_WAVES * 16 * Q_RT;        // output rows per workgroup
constexpr int Q_LUT = 256 * 128;                   // byte -> 5 fp4 codes, one copy per bank
constexpr int Q_OPS = 4 * 2 * 2 * 2048;            // operands of a window: 4 instructions x 2 token tiles x 2 pieces x 2 KiB
constexpr int Q_ABUF = Q_OPS + 2 * 64 * 4;         // ... and the block scales: per token tile one dword per lane (byte j = instruction j)
constexpr int Q_FM = Q_LUT + 2 * Q_ABUF;           // the lanes' digit masks of the 4 instructions in which a group ends: 4 x 64 x 16 bytes
constexpr int Q_XS = Q_FM + 4 * 1024;              // per wave, a transit area for the raw activations of its staging item: 16 token rows x 176 bytes
constexpr int Q_XPITCH = 176, Q_XWAVE = 16 * Q_XPITCH;
constexpr int Q_SC = Q_XS + Q_WAVES * Q_XWAVE;     // the scale ring: 2 slots of [512 rows][8 scales] as stored
constexpr int q_lds_bytes(int scale_bytes) { return Q_SC + 2 * Q_ROWS * 8 * scale_bytes; }  // 142,336 (16-bit scales) / 158,720 (float32)

// Group boundaries inside the 8 instructions J of a chunk: instruction J holds the chunk's packed bytes 16 J .. 16 J + 15;
// groups end inside bytes 25 (3 of its digits belong to the first group), 51 (1), 76 (4), 102 (2).
__device__ __forceinline__ constexpr int q_split_byte(int J) { return J == 1 ? 9 : J == 3 ? 3 : J == 4 ? 12 : J == 6 ? 6 : -1; }
__device__ __forceinline__ constexpr int q_split_digits(int J) { return J == 1 ? 3 : J == 3 ? 1 : J == 4 ? 4 : J == 6 ? 2 : 0; }

template <int ACT, int SDT>
__global__ __launch_bounds__(Q_THREADS, 2) void k_gemm_tq1(GemmArgs a) {
  constexpr int XB = ACT == BP_BF16 ? 2 : 1;   // bytes per activation
  constexpr int SB = SDT == BP_F32 ? 4 : 2;

  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, kb = lane >> 4;
  const int row_blocks = (int)((a.N + Q_ROWS - 1) / Q_ROWS);
  int wg_block;
  const TileRef tr = tile_of_workgroup(a, blockIdx.x, row_blocks, wg_block);
  if (!tr.live) return;  // uniform for the workgroup
  const int64_t e = tr.e, tok0 = tr.tok0, o1 = tr.o1;
  const int ntok = (int)(o1 - tok0 < 32 ? o1 - tok0 : 32);
  const bool two = ntok > 16;  // the second token tile holds tokens
  const int64_t n_base = (int64_t)wg_block * Q_ROWS;
  const int64_t n_wave = n_base + wave * (16 * Q_RT);

  // ---- the byte table: entry v = digits d0..d4 of v as fp4 codes (-1 -> 0xA, 0 -> 0, +1 -> 0x2) in nibbles 0..4, entry
  // v copy c at 128 v + 4 c (a lane reads copy lane % 32)
  if (threadIdx.x < 256) {
    unsigned v = threadIdx.x, ent = 0;
    if (v < 243) {
#pragma unroll
      for (int d = 0; d < 5; ++d) {
        const unsigned q = v / 3, dig = v - 3 * q;
        ent |= (dig == 0 ? 0xAu : dig == 2 ? 0x2u : 0u) << (4 * d);
        v = q;
      }
    }
    *(lds_u32*)(128 * threadIdx.x) = ent;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < 256 * 32; idx += Q_THREADS)
    if (idx & 31) *(lds_u32*)(4 * idx) = *(const lds_u32*)(128 * (idx >> 5));

  const int nwin = (int)((a.K + 319) / 320);  // 64-byte windows of a row that hold digits
  const int gs = a.group == 256 ? 1 : 0;      // scale groups of 256: two 128-wide work groups share a scale

  // ---- staging of the activation operands: thread = (token m of 16, block kb of 4) of instruction sj, token tile stt
  const int stt = wave & 1, sj = wave >> 1;
  const bool stage_on = stt == 0 || two;
  int srow = 16 * stt + r16;
  if (srow >= ntok) srow = ntok - 1;  // rows past the expert's tokens repeat its last one (their results are not stored)
  const int64_t tile_bytes = (int64_t)ntok * a.K * XB;
  const __amdgpu_buffer_rsrc_t xrs = make_rsrc((const unsigned char*)a.x + tok0 * a.K * XB, tile_bytes);
  // Loads are laid out for the memory pipeline, not for the conversion: lane (m, q) takes the 16-byte pieces q, q + 4, q + 8
  // of token m's 160 bytes (int8: 80), so four lanes cover 64 consecutive bytes of a row; the pieces go through the wave's
  // transit area in LDS, from which lane (m, kb) reads back the 20 activations of its block.
  constexpr int XP = ACT == BP_BF16 ? 3 : 2;   // 16-byte pieces per lane
  constexpr int XE = ACT == BP_BF16 ? 8 : 16;  // activations per piece
  u32x4 xr[XP];
  auto stage_load = [&](int s) {
    if (!stage_on) return;
    const int64_t k0 = 320 * (int64_t)s + 80 * sj;
#pragma unroll
    for (int i = 0; i < XP; ++i) {
      const int piece = 4 * i + kb;
      const int64_t k = k0 + XE * piece;  // K is a multiple of 16: a piece lies inside the row or past it
      const bool ok = piece * XE < 80 && k < a.K;
      const unsigned o = ok ? (unsigned)(((int64_t)srow * a.K + k) * XB) : 0xfffffff0u;  // (past the buffer: reads zeros, no memory access)
      xr[i] = buf_load16(xrs, o, 0u);
    }
  };
  auto stage_store = [&](int buf) {
    if (!stage_on) return;
    const unsigned xs = (unsigned)(Q_XS + wave * Q_XWAVE + r16 * Q_XPITCH);
#pragma unroll
    for (int i = 0; i < XP; ++i)
      if ((4 * i + kb) * XE < 80) *(lds_u32x4*)(xs + 16u * (unsigned)(4 * i + kb)) = xr[i];
    float y[20];
    if (ACT == BP_BF16) {
#pragma unroll
      for (int d = 0; d < 5; ++d) {  // (the wave's own LDS accesses are executed in order)
        const u32x2 v = *(const lds_u32x2*)(xs + 40u * kb + 8u * d);
        y[4 * d] = __uint_as_float(v.x << 16);
        y[4 * d + 1] = __uint_as_float(v.x & 0xffff0000u);
        y[4 * d + 2] = __uint_as_float(v.y << 16);
        y[4 * d + 3] = __uint_as_float(v.y & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int d = 0; d < 5; ++d) {
        const unsigned v = *(const lds_u32*)(xs + 20u * kb + 4u * d);
#pragma unroll
        for (int i = 0; i < 4; ++i) y[4 * d + i] = (float)(int)(signed char)((v >> (8 * i)) & 0xffu);
      }
    }
    unsigned mx = 0;
#pragma unroll
    for (int i = 0; i < 20; ++i) {
      const unsigned v = __float_as_uint(y[i]) & 0x7fffffffu;
      mx = mx > v ? mx : v;
    }
    const int ex = (int)(mx >> 23);
    int sh = 134 - ex;  // brings the block's largest magnitude into [128, 256)
    sh = sh > 126 ? 126 : sh;
    float mult = __uint_as_float((unsigned)(127 + sh) << 23);
    if (ex == 255) mult = __uint_as_float(0x7fc00000u);  // a NaN or an infinity in the block: every slot becomes NaN
    u32x4 blk[2][2];  // [piece][w / 2]: the 8 slots of packed bytes w and w + 1
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      float v[6];
#pragma unroll
      for (int i = 0; i < 5; ++i) v[i] = y[5 * w + i] * mult;
      v[5] = 0.f;
      unsigned p0[2] = {0u, 0u}, p1[2] = {0u, 0u};
#pragma unroll
      for (int i = 0; i < 6; i += 2) {
        const int c0 = __builtin_amdgcn_cvt_pk_fp8_f32(v[i], v[i + 1], 0, false);
        const float r0 = v[i] - __builtin_amdgcn_cvt_f32_fp8(c0, 0), r1 = v[i + 1] - __builtin_amdgcn_cvt_f32_fp8(c0, 1);
        const int c1 = __builtin_amdgcn_cvt_pk_fp8_f32(r0, r1, 0, false);
        p0[i >> 2] |= ((unsigned)c0 & 0xffffu) << (16 * ((i >> 1) & 1));
        p1[i >> 2] |= ((unsigned)c1 & 0xffffu) << (16 * ((i >> 1) & 1));
      }
      blk[0][w >> 1][2 * (w & 1)] = p0[0];
      blk[0][w >> 1][2 * (w & 1) + 1] = p0[1];
      blk[1][w >> 1][2 * (w & 1)] = p1[0];
      blk[1][w >> 1][2 * (w & 1) + 1] = p1[1];
    }
    const unsigned ab = (unsigned)(Q_LUT + buf * Q_ABUF);
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const unsigned ob = ab + (unsigned)(((sj * 2 + stt) * 2 + p) * 2048);
#pragma unroll
      for (int b = 0; b < 2; ++b)  // bytes w = 2 b, 2 b + 1 -> A lane quarter 2 (kb % 2) + b, half kb / 2
        *(lds_u32x4*)(ob + (unsigned)((((2 * (kb & 1) + b) * 2 + (kb >> 1)) * 256) + r16 * 16)) = blk[p][b];
    }
    *(__attribute__((address_space(3))) unsigned char*)(ab + Q_OPS + (unsigned)((stt * 64 + lane) * 4 + sj)) = (unsigned char)(127 - sh);
  };

  // ---- the lanes' masks for the four instructions in which a scale group ends (the digits of the first group), in LDS
  if (wave == 0) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int J = q == 0 ? 1 : q == 1 ? 3 : q == 2 ? 4 : 6;
      u32x4 m;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int idx = 4 * kb + w;
        m[w] = idx < q_split_byte(J) ? 0xffffffffu : idx == q_split_byte(J) ? (1u << (4 * q_split_digits(J))) - 1u : 0u;
      }
      *(lds_u32x4*)(unsigned)(Q_FM + q * 1024 + lane * 16) = m;
    }
  }
  const unsigned lane4 = (unsigned)(lane & 31) << 2;
  const unsigned alane = (unsigned)(kb * 512 + r16 * 16);
  int ones = 0x7f7f7f7f;  // operand B's block scales: 2^0
  asm volatile("" : "+v"(ones));

  auto all_terms = [&](auto tt_c) {
    constexpr int TT = decltype(tt_c)::value;  // token tiles processed
    f32x4 total[Q_RT][TT];
#pragma unroll
    for (int r = 0; r < Q_RT; ++r)
#pragma unroll
      for (int t = 0; t < TT; ++t) total[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    for (int term = 0; term < a.n_terms; ++term) {
      // the expert's rows as a buffer that ends with the tensor; dword-aligned base, per-lane row offset
      const unsigned char* wbeg = a.packed[term];
      const unsigned char* expert_rows = wbeg + e * a.N * a.Kp;
      const unsigned mis = (unsigned)((uintptr_t)expert_rows & 3);
      const __amdgpu_buffer_rsrc_t wrs = make_rsrc(expert_rows - mis, (wbeg + a.E * a.N * a.Kp) - (expert_rows - mis));
      const unsigned voff = mis + (unsigned)r16 * (unsigned)a.Kp + 16u * kb;  // (rows start at any byte: the 16-byte loads are not aligned)
      unsigned wrow[Q_RT];  // byte offset of the row tile's first row (a tile past N repeats the wave's first tile and is not stored)
#pragma unroll
      for (int r = 0; r < Q_RT; ++r) {
        int64_t row = n_wave + 16 * r;
        if (row >= a.N) row = n_wave < a.N ? n_wave : 0;
        wrow[r] = (unsigned)(row * a.Kp);
      }
      u32x4 W[Q_RT];
      // The last row of the tensor in its last window: a 16-byte load that reaches past the end of the buffer loses the
      // dwords that straddle the end, valid bytes included, so the one wave that holds that row loads it byte by byte
      // (every byte is range-checked by itself).
      const bool tail_wave = e == a.E - 1 && n_wave < a.N && n_wave + 16 * Q_RT >= a.N;
      auto fetch_w = [&](int s, int r) {  // (r: compile-time constant after unrolling)
        const int ss = s < nwin ? s : nwin - 1;
        W[r] = buf_load16(wrs, voff, wrow[r] + 64u * (unsigned)ss);
        if (tail_wave && ss == nwin - 1 && n_wave + 16 * r + 16 == a.N) {  // uniform: the tile that ends with row N - 1
          u32x4 v = {0u, 0u, 0u, 0u};
#pragma unroll
          for (int i = 0; i < 16; ++i)
            v[i >> 2] |= (unsigned)(unsigned char)__builtin_amdgcn_raw_buffer_load_b8(wrs, (int)(voff + (unsigned)i), (int)(wrow[r] + 64u * (unsigned)ss), 0) << (8 * (i & 3));
          W[r] = v;
        }
      };

      // The scales go through LDS as stored, in blocks of 8 consecutive entries per row (thread = row, one or two 16-byte
      // loads every 8 groups), two blocks resident: block b + 2 replaces block b at the end of a chunk's second window, when
      // only a chunk's first two groups can still lie in block b, and those are added in the chunk's first window.
      const unsigned char* sbeg = (const unsigned char*)a.w_scale[term];
      const unsigned char* expert_scales = sbeg + e * a.N * a.G * SB;
      const __amdgpu_buffer_rsrc_t srs = make_rsrc(expert_scales, (sbeg + a.E * a.N * a.G * SB) - expert_scales);
      const int64_t my_row = n_base + threadIdx.x;
      const unsigned my_scales = my_row < a.N ? (unsigned)(my_row * a.G * SB) : 0xfffffff0u;  // rows past N: zeros
      constexpr int SLOT = Q_ROWS * 8 * SB;
      u32x4 sq[SB / 2];
      int sc_loaded = 0;  // highest block in LDS (uniform)
      auto scale_load = [&](int b) {
#pragma unroll
        for (int i = 0; i < SB / 2; ++i) sq[i] = buf_load16(srs, my_scales == 0xfffffff0u ? my_scales : my_scales + (unsigned)(b * 8 * SB + 16 * i), 0u);
      };
      auto scale_store = [&](int b) {
#pragma unroll
        for (int i = 0; i < SB / 2; ++i) *(lds_u32x4*)(unsigned)(Q_SC + (b & 1) * SLOT + (int)threadIdx.x * (8 * SB) + 16 * i) = sq[i];
      };
      auto last_block_of = [&](int c) { return (int)(((5 * (int64_t)c + 4) >> gs) >> 3); };

      // ---- prologue of the term: window 0's operands and chunk 0's scales into LDS, window 0's weights on their way
      __syncthreads();  // (the previous term's last window has been read by every wave)
      stage_load(0);
      scale_load(0);
#pragma unroll
      for (int r = 0; r < Q_RT; ++r) fetch_w(0, r);
      stage_store(0);
      scale_store(0);
      __syncthreads();

      f32x4 C[Q_RT][TT];
#pragma unroll
      for (int r = 0; r < Q_RT; ++r)
#pragma unroll
        for (int t = 0; t < TT; ++t) C[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

      // one window: H = 0 / 1, the first / second 64 bytes of chunk c
      auto window = [&](int c, auto h_c) {
        constexpr int H = decltype(h_c)::value;
        const int s = 2 * c + H;
        const unsigned ab = (unsigned)(Q_LUT + (s & 1) * Q_ABUF);
        const unsigned sb = (unsigned)(Q_SC + (wave * (16 * Q_RT) + r16) * (8 * SB));
        // this window's bytes: shifted to the row's alignment, then transposed between the row's four lanes, so that
        // dword j of lane quarter kb holds the window's bytes 16 j + 4 kb .. + 3
        unsigned D[Q_RT][4];
#pragma unroll
        for (int r = 0; r < Q_RT; ++r) {
          unsigned d0 = W[r].x, d1 = W[r].y, d2 = W[r].z, d3 = W[r].w;
          const auto s02 = __builtin_amdgcn_permlane32_swap(d0, d2, false, false);
          const auto s13 = __builtin_amdgcn_permlane32_swap(d1, d3, false, false);
          const auto s01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
          const auto s23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
          D[r][0] = s01[0];
          D[r][1] = s01[1];
          D[r][2] = s23[0];
          D[r][3] = s23[1];
        }
        // next window: weights into the registers just consumed, activations (converted and stored when this window's
        // instructions have been issued), and at the end of a chunk the next chunk's scales
        const bool more = s + 1 < nwin;
        const bool new_scales = H == 1 && more && last_block_of(c + 1) > sc_loaded;  // (at most one block further)
        // The next window's loads are spread over this window's instructions (weights: into the registers just consumed):
        // issued in one burst by all eight waves they fill the memory pipeline's queues, and a wave that cannot issue a
        // load cannot issue anything else either.
        if (more) stage_load(s + 1);
        int sa[TT];
#pragma unroll
        for (int t = 0; t < TT; ++t) sa[t] = (int)*(const lds_u32*)(ab + Q_OPS + (unsigned)((t * 64 + lane) * 4));

        auto flush = [&](int g) {  // group g of the chunk is complete: its sums under its scales
          const int si = (int)((5 * (int64_t)c + g) >> gs);  // the group's scale: entry si of the row, in slot (si / 8) % 2
          const unsigned at = sb + (unsigned)(((si >> 3) & 1) * SLOT + (si & 7) * SB);
#pragma unroll
          for (int r = 0; r < Q_RT; ++r) {
            float sc;
            if (SDT == BP_F32) sc = __uint_as_float(*(const lds_u32*)(at + (unsigned)(16 * r * 8 * SB)));
            else {
              const unsigned raw = *(const __attribute__((address_space(3))) uint16_t*)(at + (unsigned)(16 * r * 8 * SB));
              sc = SDT == BP_F16 ? f16_bits_to_f32((uint16_t)raw) : __uint_as_float(raw << 16);
            }
#pragma unroll
            for (int t = 0; t < TT; ++t) {
#pragma unroll
              for (int i = 0; i < 4; ++i) total[r][t][i] += sc * C[r][t][i];
              C[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
          }
        };
        // One instruction slot j of the window: `pre` (a share of the next window's loads and conversions), this slot's
        // table and operand reads, its matrix instructions and the scaling of a completed group.
        auto instr = [&](auto j_c, auto&& pre) {
          constexpr int j = decltype(j_c)::value, J = 4 * H + j;
          constexpr int SPLIT = q_split_byte(J) >= 0;
          constexpr int Q = J == 1 ? 0 : J == 3 ? 1 : J == 4 ? 2 : 3;  // (index into fm)
          auto& tot = total;
          pre();
          u32x4 B[Q_RT];
#pragma unroll
          for (int r = 0; r < Q_RT; ++r)
#pragma unroll
            for (int w = 0; w < 4; ++w) {
              const unsigned at = (((D[r][j] >> (8 * w)) & 0xffu) << 7) | lane4;
              B[r][w] = *(const lds_u32*)at;
            }
          i32x8 A[TT][2];
#pragma unroll
          for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int p = 0; p < 2; ++p) {
              const unsigned at = ab + (unsigned)(((j * 2 + t) * 2 + p) * 2048) + alane;
              const u32x4 lo = *(const lds_u32x4*)at, hi = *(const lds_u32x4*)(at + 256);
              A[t][p] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            }
          u32x4 fm = {0u, 0u, 0u, 0u};
          if (SPLIT) fm = *(const lds_u32x4*)(unsigned)(Q_FM + Q * 1024 + lane * 16);
          auto multiply = [&](auto part_c) {  // part 0: all digits (or those of the first group), part 1: those of the second group
            constexpr int PART = decltype(part_c)::value;
#pragma unroll
            for (int p = 0; p < 2; ++p)
#pragma unroll
              for (int r = 0; r < Q_RT; ++r) {
                u32x4 b = B[r];
                if (SPLIT) {
#pragma unroll
                  for (int w = 0; w < 4; ++w) b[w] = PART == 0 ? b[w] & fm[w] : b[w] ^ (b[w] & fm[w]);
                }
                const i32x8 B8 = {(int)b.x, (int)b.y, (int)b.z, (int)b.w, 0, 0, 0, 0};
#pragma unroll
                for (int t = 0; t < TT; ++t)
                  C[r][t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[t][p], B8, C[r][t], 0 /* A: E4M3 */, 4 /* B: E2M1 */, j, sa[t], 0, ones);
              }
          };
          __builtin_amdgcn_sched_barrier(0);
          multiply(QC<0>{});
          if (SPLIT) {
            flush(J == 1 ? 0 : J == 3 ? 1 : J == 4 ? 2 : 3);
            multiply(QC<1>{});
          }
          if (J == 7) flush(4);
          // (an opaque use: without it the compiler sinks the matrix instructions - pure, and read only by later blocks -
          // below the conversion of the next window's activations, with every operand of the window held in registers)
#pragma unroll
          for (int r = 0; r < Q_RT; ++r)
#pragma unroll
            for (int t = 0; t < TT; ++t) {
              asm volatile("" : "+v"(C[r][t]));
              if (SPLIT || J == 7) asm volatile("" : "+v"(tot[r][t]));
            }
        };
        __builtin_amdgcn_sched_barrier(0);
        instr(QC<0>{}, [&] {});
        __builtin_amdgcn_sched_barrier(0);
        instr(QC<1>{}, [&] { if (more) { fetch_w(s + 1, 0); fetch_w(s + 1, 1); } });
        __builtin_amdgcn_sched_barrier(0);
        // (the conversion is vector-ALU work: the two waves that share a SIMD have it in different slots)
        instr(QC<2>{}, [&] {
          if (more) { fetch_w(s + 1, 2); fetch_w(s + 1, 3); }
          if (new_scales) scale_load(sc_loaded + 1);
          if (more && wave < 4) stage_store((s + 1) & 1);
        });
        __builtin_amdgcn_sched_barrier(0);
        instr(QC<3>{}, [&] {
          if (more && wave >= 4) stage_store((s + 1) & 1);
          if (new_scales) {
            scale_store(sc_loaded + 1);
            ++sc_loaded;
          }
        });
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
      };

      const int nchunks = (nwin + 1) >> 1;
      for (int c = 0; c < nchunks; ++c) {
        window(c, QC<0>{});
        if (2 * c + 1 < nwin) window(c, QC<1>{});  // uniform
      }
      // a last chunk without its second window: groups 0 and 1 have been added; group 2 onwards lies past K (their sums are 0)
    }

    // ---- epilogue: lane holds tokens 4 kb + i of each token tile, output row n_wave + 16 r + r16
#pragma unroll
    for (int t = 0; t < TT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tk = 16 * t + 4 * kb + i;
        if (tk < ntok) {
          const int64_t tok = tok0 + tk;
          const float xs = ACT == BP_I8 ? a.x_scale[tok] : 1.0f;
#pragma unroll
          for (int r = 0; r < Q_RT; ++r) {
            const int64_t row = n_wave + 16 * r;
            if (row < a.N) {
              float* o = a.out + tok * a.N + row + r16;
              *o = (a.overwrite ? 0.f : *o) + total[r][t][i] * xs;
            }
          }
        }
      }
    }
  };
  if (two) all_terms(QC<2>{});
  else all_terms(QC<1>{});
}

template <int ACT, int SDT>
int launch_gemm_tq1_k(const GemmArgs& a, hipStream_t s, const char* name) {
  if (const int rc = raise_lds_limit<k_gemm_tq1<ACT, SDT>>(q_lds_bytes(SDT == BP_F32 ? 4 : 2))) return rc;
  const int64_t row_blocks = (a.N + Q_ROWS - 1) / Q_ROWS;
  const int64_t wgs = tile_workgroups(a, row_blocks);
  if (wgs < 0) return BP_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)wgs, 1, 1);
  note_kernel(name);
  hipLaunchKernelGGL((k_gemm_tq1<ACT, SDT>), grid, dim3(Q_THREADS), q_lds_bytes(SDT == BP_F32 ? 4 : 2), s, a);
  return check_launch(name);
}

}  // namespace

// Preconditions (beyond mfma_supports: groups of 128 or 256, K % 256 == 0, K >= 1024, N % 16 == 0, 16-byte aligned x):
// bf16 or int8 activations; 4-byte aligned scale rows; K small enough for 32-bit offsets into a 32-token activation tile.
// BP_ERR_UNSUPPORTED (no message): the caller falls back to its other kernels.
int launch_gemm_tq1(const GemmArgs& a, hipStream_t s) {
  if (a.stage && tuning().tq2g != 'b') {  // with a workspace: one matrix instruction per scale group over converted activations (bp_gemm_tq2f.hip; development: BP_TUNE_TQ2G=bf16 keeps this file's kernel)
    const int rc = launch_gemm_tq2f(a, s);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  if (a.x_dtype != BP_BF16 && a.x_dtype != BP_I8) return BP_ERR_UNSUPPORTED;
  if (a.K > ((int64_t)1 << 24) || a.N * a.Kp > ((int64_t)1 << 31) - 4096) return BP_ERR_UNSUPPORTED;
  if ((a.max_rows + 31) / 32 > 65535) return BP_ERR_UNSUPPORTED;
  if (a.x_dtype == BP_BF16) {
    if (a.scale_dtype == BP_F16) return launch_gemm_tq1_k<BP_BF16, BP_F16>(a, s, "gemm_tq1_bf16");
    if (a.scale_dtype == BP_BF16) return launch_gemm_tq1_k<BP_BF16, BP_BF16>(a, s, "gemm_tq1_bf16");
    return launch_gemm_tq1_k<BP_BF16, BP_F32>(a, s, "gemm_tq1_bf16");
  }
  if (a.scale_dtype == BP_F16) return launch_gemm_tq1_k<BP_I8, BP_F16>(a, s, "gemm_tq1_i8");
  if (a.scale_dtype == BP_BF16) return launch_gemm_tq1_k<BP_I8, BP_BF16>(a, s, "gemm_tq1_i8");
  return launch_gemm_tq1_k<BP_I8, BP_F32>(a, s, "gemm_tq1_i8");
}

}  // namespace bp

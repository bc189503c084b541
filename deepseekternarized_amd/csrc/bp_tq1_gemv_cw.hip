// TQ1 decode GEMV of large calls: the rows streamed through LDS tile by tile by loader waves, a chunk of the token's
// fp8 operand in the registers of each multiplier wave (v_mfma_f32_16x16x128_f8f6f4, weights as fp4). The arithmetic
// (three or two fp8 pieces per activation under a power-of-two prescale per group, scale groups as rows of operand A,
// the byte table) is that of bp_tq1_gemv_fp4.hip, whose head describes it; contract as everywhere
// (boilerplate/kernels/ternary_cuda.py:58-63).
#include "bp_tq1_fp4.h"

namespace bp {
namespace {

// ---- One token row per expert, the rows streamed through LDS tile by tile: "a chunk per wave" -------------------------
//
// The kernel above lets every wave walk along its own 16 rows: a wave load is 16 rows x 64 bytes (rows of Kp bytes start
// at any byte, so each of the 16 pieces straddles memory lines that the wave comes back to chunks later), and operand A
// is read from LDS once per matrix instruction - 8 x the packed bytes. Here a workgroup of 16 waves walks over tiles of
// 16 rows together, with two kinds of waves:
//  * loaders request a tile's 16 x Kp bytes as 4 rows x 256 bytes per wave load (a lane takes 16 bytes at a dword-aligned
//    address; LPW loads per loader and tile, the tile's scales - 16 x G x 2 bytes, contiguous - among them), two tiles
//    ahead, and park them in tile buffers in LDS (row n at n x pitch, shifted by the row's misalignment of 0..3 bytes);
//  * multipliers read a tile back as the matrix instruction wants it (row n = lane % 16, the 16-byte quarters of a 64-byte
//    window across lanes / 16, plus the dword that follows for the realignment). Wave c of a group keeps chunk c of the
//    token's operand A in registers (8 instructions x 8 registers) and multiplies chunk c of every tile: no operand A
//    reads in the loop. A group is nchunks multipliers and its loaders; groups walk over their own tiles (tile index =
//    group mod groups);
//  * a multiplier's 16 partial sums of a tile (one per row) go to LDS, and the group's loaders (token t by loader t mod their number) add the chunks' sums
//    in a fixed order and adds the result to the row's entry of the workgroup's outputs, which wait in LDS too: read
//    from memory when the workgroup starts, written back once after the last term.
// A barrier hands over TPB tiles: two where four tile buffers fit beside the table (the loaders' waits for memory and
// the multipliers' work vary from tile to tile: the fewer the meeting points, the less is waited), else one with two
// buffers. The buffers that the loaders fill were multiplied before the previous barrier. The tile buffers take the
// place of the operand A tiles once those are in registers.
constexpr int CW_WAVES = 16;
constexpr int CW_LUT_BYTES = 256 * 256;  // byte -> 5 fp4 codes, 64 copies: entry v copy c at 256 v + 4 c
constexpr int CW_STAGE_PER_THREAD = 4;    // outputs of a workgroup per thread at most (they wait in LDS from the first barrier to the end)
// A row's image in a tile buffer: up to 3 bytes of misalignment, the row's Kp bytes and the dword after them, in whole
// 16-byte pieces, at a pitch that is an odd number of pieces (16 rows: 16 different groups of 4 banks). What a
// multiplier reads past a row's image in its last chunk (the next row's bytes, or what follows the buffer) meets
// activations that are 0.
constexpr int cw_pitch(int64_t Kp) {
  const int pieces = (int)((Kp + 3 + 4 + 15) / 16);
  return 16 * (pieces | 1);
}
constexpr int cw_colblks(int64_t Kp) { return (int)((Kp + 3 + 255) / 256); }  // wave loads of 4 rows x 256 bytes per 4 rows
constexpr int64_t cw_buffer_bytes(int64_t Kp, int64_t G, int64_t scale_bytes) { return 16 * (int64_t)cw_pitch(Kp) + 16 * G * scale_bytes; }

// LPW: wave loads of packed bytes per loader and tile; TPB: tiles per barrier. NTOK = 2: a pair of token rows per expert
// (rows first_row, first_row + 1), as in the kernel above: two fp8 pieces per activation, one matrix instruction serves
// both tokens (row 4 s + 2 t + p of operand A = piece p of token t in group slot s), an accumulator tile per 64-byte window,
// and a multiplier's registers hold the pair's chunk (the same 8 x 8 registers).
template <int SDT, int LPW, int TPB, int NTOK = 1>
__global__ __launch_bounds__(CW_WAVES * 64) void k_tq1_gemv_cw(GemmArgs a, int nchunks, int groups, int tiles_per_wg, int first_row) {
  static_assert(NTOK == 1 || NTOK == 2 || NTOK == 4, "one token row per expert, a pair, or four");
  // NTOK = 4: the multipliers read their rows' bytes piece by piece (byte map 1 of bp_tq1_fp4.h), so that a matrix
  // instruction covers 80 consecutive digits = at most two scale groups and the 16 rows of operand A are 2 group slots x
  // 4 tokens x 2 pieces; four accumulator tiles per chunk. The four tokens' tiles (108 KiB at K = 7168) are built from
  // LDS address 0, where the table goes once the multipliers have their operand in registers.
  constexpr bool M4 = NTOK == 4;
  constexpr int WAVES = CW_WAVES, THREADS = WAVES * 64, NB = 2 * TPB, PC = f4_pieces(NTOK), SB = SDT == BP_F32 ? 4 : 2;
  constexpr int F4_INV_OFF = F4Tile<PC>::INV_OFF, F4_CHUNK_BYTES = F4Tile<PC>::CHUNK_BYTES, AT = CW_LUT_BYTES;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, kb = lane >> 4;
  const int64_t e = blockIdx.y;
  const int64_t o0 = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  const int64_t tok = o0 + first_row;
  if (tok >= o1) return;  // (uniform: an expert without a token row in this launch)
  const int ntok = o1 - tok < NTOK ? (int)(o1 - tok) : NTOK;
  float xsc[NTOK];
#pragma unroll
  for (int tt = 0; tt < NTOK; ++tt) xsc[tt] = a.x_dtype == BP_I8 && tt < ntok ? a.x_scale[tok + tt] : 1.f;
  const int gs = a.group == 256 ? 1 : 0;

  // ---- roles (wave-uniform): multiplier of chunk c in group grp, or loader number lidx of the group's lpg loaders
  const int active = groups * nchunks, extra = wave - active, lpg = (WAVES - active) / groups;
  const bool multiplier = wave < active, loader = !multiplier && extra < lpg * groups;
  const int grp = multiplier ? wave / nchunks : extra % groups;
  const int c = multiplier ? wave - grp * nchunks : 0;
  const int lidx = multiplier ? 0 : extra / groups;

  // ---- LDS behind the table: per group NB tile buffers (16 rows at `pitch`, then the tile's scales), then the partial sums
  const int colblks = cw_colblks(a.Kp), pitch = cw_pitch(a.Kp);
  const int scb = (int)(16 * a.G * SB);  // a tile's scales: 16 rows x G entries, contiguous
  const int buf_bytes = 16 * pitch + scb;
  const unsigned gbase = (unsigned)(AT + grp * NB * buf_bytes);
  const unsigned red = (unsigned)(AT + groups * NB * buf_bytes + grp * NB * nchunks * 64 * NTOK);  // [tile % NB][chunk][token][row]
  const int nl = 4 * colblks, ns = (scb + 1023) >> 10;  // wave loads of a tile: packed bytes, scales
  const int64_t tiles = a.N / 16;
  const int64_t tile0 = (int64_t)blockIdx.x * tiles_per_wg;
  const int64_t tile_end = tile0 + tiles_per_wg < tiles ? tile0 + tiles_per_wg : tiles;
  const int n_iter = (tiles_per_wg + groups - 1) / groups;  // tiles of a group
  const int n_int = (n_iter + TPB - 1) / TPB;                 // barriers: TPB tiles each
  auto tile_of = [&](int t) -> int64_t { return tile0 + (int64_t)t * groups + grp; };
  // ---- the workgroup's outputs, [tile of the workgroup][token][row] float32, behind the buffers and sums (and behind the
  // operand A tiles, which are built in the buffers' place): read from memory now, parked in LDS before the first
  // barrier, added to there tile by tile, and written back once after the last term - no access to the outputs in the loop.
  const int stream_bytes = groups * NB * (buf_bytes + nchunks * 64 * NTOK), build_bytes = nchunks * NTOK * F4_CHUNK_BYTES;
  const unsigned stage = M4 ? (unsigned)(AT + stream_bytes > build_bytes ? AT + stream_bytes : build_bytes)
                            : (unsigned)(AT + (stream_bytes > build_bytes ? stream_bytes : build_bytes));
  const int n_stage = (int)(tile_end - tile0) * 16 * NTOK;  // (at most CW_STAGE_PER_THREAD x the workgroup's threads: the launcher's bound)
  auto out_index = [&](int o) -> int64_t { return (tok + ((o >> 4) % NTOK)) * a.N + (tile0 + (o >> 4) / NTOK) * 16 + (o & 15); };
  float was[CW_STAGE_PER_THREAD];
#pragma unroll
  for (int u = 0; u < CW_STAGE_PER_THREAD; ++u) {
    const int o = (int)threadIdx.x + u * THREADS;
    was[u] = o < n_stage && ((o >> 4) % NTOK) < ntok ? a.out[out_index(o)] : 0.f;
  }

  // ---- loaders: state of the current term (the expert's rows and scales as buffers of their own: a tile past N reads
  // zeros) and the wave's loads of a tile: LPW of the nl wave loads of packed bytes (li = i * lpg + lidx: rows
  // 4 (li % 4) .. + 3, bytes 256 (li / 4) .. + 255 of the rows' LDS images; what depends on li is uniform and goes into
  // the loads' scalar offsets, so one lane offset serves all of them) and one of the ns wave loads of the scales
  __amdgpu_buffer_rsrc_t wrs = make_rsrc(a.packed[0], 0), srs = wrs;
  unsigned w_lane = 0, w_last = 0, s_lane = 0x7ffffff0u;  // lane offsets of the loads (past the buffer: zeros, no memory access)
  const unsigned d_lane = (unsigned)(kb * pitch + 16 * r16), ds_lane = (unsigned)(16 * pitch + 16 * (lidx * 64 + lane));
  const bool put_s = loader && lidx < ns && 16 * (lidx * 64 + lane) < scb;
  u32x4 ring[2][LPW + 1];
  auto slot_li = [&](int i) { return i * lpg + lidx; };
  auto setup_term = [&](int term) {
    const unsigned char* expert_rows = a.packed[term] + e * a.N * a.Kp;
    const unsigned mis = (unsigned)((uintptr_t)expert_rows & 3);
    wrs = make_rsrc(expert_rows - mis, whole_dwords(a.N * a.Kp + mis));
    srs = make_rsrc((const unsigned char*)a.w_scale[term] + e * a.N * a.G * SB, a.N * a.G * SB);  // (dword-aligned: checked by the host)
    const unsigned ro = mis + (unsigned)kb * (unsigned)a.Kp;
    w_lane = (ro & ~3u) + 16u * (unsigned)r16;  // (rows 4 apart are a multiple of 4 bytes apart)
    // (the last block of 256 bytes: only the pieces that hold bytes of the row)
    w_last = 256 * (colblks - 1) + 16 * r16 < (int)(ro & 3u) + (int)a.Kp ? w_lane : 0x7ffffff0u;
    s_lane = put_s ? (unsigned)(16 * (lidx * 64 + lane)) : 0x7ffffff0u;
  };
  const unsigned step_w = (unsigned)(16 * a.Kp), step_s = (unsigned)scb;  // a tile's bytes
  auto request = [&](int t, auto slot_c) {  // the loads of the tile of iteration t
    constexpr int slot = decltype(slot_c)::value;
    const int64_t tile = tile_of(t);
    const bool live = loader && tile < tiles;
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int li = slot_li(i);
      const unsigned so = (unsigned)tile * step_w + (unsigned)(4 * (li & 3)) * (unsigned)a.Kp + 256u * (unsigned)(li >> 2);
      ring[slot][i] = buf_load16(wrs, (li >> 2) == colblks - 1 ? w_last : w_lane, live && li < nl ? so : 0x7ffffff0u);
    }
    ring[slot][LPW] = buf_load16(srs, s_lane, live ? (unsigned)tile * step_s : 0x7ffffff0u);
  };
  auto park = [&](int t, auto slot_c) {  // ... into the buffer of iteration t
    constexpr int slot = decltype(slot_c)::value;
    const unsigned wb = gbase + (unsigned)((t % NB) * buf_bytes);
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const int li = slot_li(i);
      if (loader && li < nl) {  // (uniform; in a row's last block of 256 bytes only the pieces that hold bytes of the row: the next row's image follows)
        if ((li >> 2) < colblks - 1 || w_last != 0x7ffffff0u) *(lds_u32x4*)(wb + (unsigned)(4 * (li & 3) * pitch + 256 * (li >> 2)) + d_lane) = ring[slot][i];
      }
    }
    if (put_s) *(lds_u32x4*)(wb + ds_lane) = ring[slot][LPW];
  };
  // ---- the byte table, one copy per lane (64 banks: no two lanes of a wave share one): entry v = digits d0..d4 of v as
  // fp4 codes in nibbles 0..4, at 256 v + 4 lane - an address that one byte permute makes from a packed byte and 4 lane
  auto build_table = [&] {
  for (int idx = threadIdx.x; idx < 256 * 16; idx += THREADS) {
    unsigned v = (unsigned)idx >> 4, ent = 0;
    if (v < 243) {
#pragma unroll
      for (int d = 0; d < 5; ++d) {
        const unsigned q = v / 3, dig = v - 3 * q;
        ent |= (dig == 0 ? 0xAu : dig == 2 ? 0x2u : 0u) << (4 * d);
        v = q;
      }
    }
    *(lds_u32x4*)(16 * idx) = u32x4{ent, ent, ent, ent};
  }
  };
  // A loader has few instructions per tile and everything waits for them: they go before those of the multipliers on
  // its SIMD. The first term's first two tiles are requested before the table and the token's tile are built.
  if (!multiplier) {
    __builtin_amdgcn_s_setprio(3);
    setup_term(0);
    request(0, IC<0>{});
    request(1, IC<1>{});
    if constexpr (!M4) build_table();
  } else if constexpr (!M4) {  // (chunk by chunk, by the multipliers; their part of the table while the activations are on their way)
    f4_build_tiles<NTOK, WAVES, AT>(a, tok, ntok, nchunks, 0, wave, lane, active, build_table);
  }
  if constexpr (M4) f4_build_tiles<NTOK, WAVES, 0, 1>(a, tok, ntok, nchunks, 0, wave, lane, WAVES);  // (all waves, where the table will be)

#pragma unroll
  for (int u = 0; u < CW_STAGE_PER_THREAD; ++u) {
    const int o = (int)threadIdx.x + u * THREADS;
    if (o < n_stage) *(lds_u32*)(stage + 4u * (unsigned)o) = __float_as_uint(was[u]);
  }
  __syncthreads();

  if (multiplier) {
    // ---- the wave's chunk of operand A (a pair: the lane's token's tile), and the inverse prescales of the lane's two
    // groups: one token: group kb and group 4, of which the lane holds piece kb; a pair: the lane's group of the first
    // window and of the second (kb and 3, 4, 2, 2 for kb = 0..3; the lanes kb = 3 hold unused rows: their sums are 0)
    i32x8 A[8];
    float inv_a[NTOK], inv_b[NTOK];
    float inv_c[2] = {0.f, 0.f};  // (M4: the lane's third group)
    const int g_w0 = M4 ? kb >> 1 : NTOK == 1 ? kb : kb < 3 ? kb : 2, g_w1 = M4 ? 2 + (kb >> 1) : NTOK == 1 ? 4 : kb == 0 ? 3 : kb == 1 ? 4 : 2;
    {
      unsigned aoff[4];
      if constexpr (M4) f4_block_offsets4(r16, kb, aoff);
      else f4_block_offsets<PC>(r16, kb, aoff);
      const unsigned cbase = (unsigned)((M4 ? 0 : AT) + c * NTOK * F4_CHUNK_BYTES);
      const unsigned mine = cbase + (M4 ? (unsigned)(((r16 >> 1) & 3) * F4_CHUNK_BYTES) : NTOK == 2 ? (unsigned)(((r16 >> 1) & 1) * F4_CHUNK_BYTES) : 0u);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const u32x4 lo = *(const lds_u32x4*)((((aoff[j >> 1] >> (16 * (j & 1))) & 0xffu) << 4) + mine);
        const u32x4 hi = *(const lds_u32x4*)((((aoff[j >> 1] >> (16 * (j & 1) + 8)) & 0xffu) << 4) + mine);
        A[j] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
      }
      const float f4th = kb == 3 ? 0.f : kb == 2 ? 1.f / 256.f : 1.f;
      if constexpr (M4) {  // the lane's two tokens 2 (kb % 2) + t; slot 0 lanes: groups 0, 2, 4, slot 1 lanes: 1, 3
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          const unsigned tile = cbase + (unsigned)((2 * (kb & 1) + t2) * F4_CHUNK_BYTES + F4_INV_OFF);
          inv_a[t2] = __uint_as_float(*(const lds_u32*)(tile + 4 * g_w0));
          inv_b[t2] = __uint_as_float(*(const lds_u32*)(tile + 4 * g_w1));
          inv_c[t2] = (kb >> 1) ? 0.f : __uint_as_float(*(const lds_u32*)(tile + 4 * 4));
          inv_a[t2 + 2] = inv_b[t2 + 2] = 0.f;
        }
      } else {
#pragma unroll
        for (int tt = 0; tt < NTOK; ++tt) {
          inv_a[tt] = __uint_as_float(*(const lds_u32*)(cbase + tt * F4_CHUNK_BYTES + F4_INV_OFF + 4 * g_w0));
          inv_b[tt] = __uint_as_float(*(const lds_u32*)(cbase + tt * F4_CHUNK_BYTES + F4_INV_OFF + 4 * g_w1)) * (NTOK == 1 ? f4th : 1.f);
        }
      }
    }
    const unsigned lane4 = (unsigned)lane << 2;
    // the lane's reads of a tile: its row's window of chunk c, and the scales of its two groups (an index past the row's
    // last group - the last chunk of a row - meets sums that are 0 and takes the last group's scale)
    const unsigned rd_w = (unsigned)(r16 * pitch + 128 * c + 16 * kb);
    const int64_t g_last = a.G - 1;
    const int64_t ga = (5 * (int64_t)c + g_w0) >> gs, gb = (5 * (int64_t)c + g_w1) >> gs;
    const unsigned rd_sa = (unsigned)(16 * pitch + r16 * (int)(a.G * SB) + SB * (int)(ga < g_last ? ga : g_last));
    const unsigned rd_sb = (unsigned)(16 * pitch + r16 * (int)(a.G * SB) + SB * (int)(gb < g_last ? gb : g_last));
    const int64_t gc = (5 * (int64_t)c + 4) >> gs;
    const unsigned rd_sc = (unsigned)(16 * pitch + r16 * (int)(a.G * SB) + SB * (int)(gc < g_last ? gc : g_last));  // (M4)
    const unsigned rd_w4 = (unsigned)(r16 * pitch + 128 * c + 4 * kb);                                             // (M4: dword kb of piece j at + 16 j)
    __syncthreads();  // (every multiplier has its operand A: the tile buffers may overwrite the tiles)
    if constexpr (M4) {
      build_table();
      __syncthreads();
    }

    for (int term = 0; term < a.n_terms; ++term) {
      const unsigned mis = (unsigned)((uintptr_t)(a.packed[term] + e * a.N * a.Kp) & 3);
      const unsigned dlt = (mis + (unsigned)r16 * (unsigned)a.Kp) & 3u;  // the lane's row starts dlt bytes into its LDS row
      auto multiply = [&](int t) {
        const unsigned rb = gbase + (unsigned)((t % NB) * buf_bytes);
        const u32x4 W0 = *(const lds_u32x4*)(rb + rd_w), W1 = *(const lds_u32x4*)(rb + rd_w + 64);
        const unsigned x0 = *(const lds_u32*)(rb + rd_w + 16), x1 = *(const lds_u32*)(rb + rd_w + 80);
        const unsigned ra = SB == 4 ? *(const lds_u32*)(rb + rd_sa) : (unsigned)*(const lds_u16*)(rb + rd_sa);
        const unsigned rbits = SB == 4 ? *(const lds_u32*)(rb + rd_sb) : (unsigned)*(const lds_u16*)(rb + rd_sb);
        // the table reads run BD instructions ahead of the matrix instructions (the scheduling barriers keep the compiler
        // from sinking them back to their uses: a wave would wait out an LDS round trip per instruction)
        constexpr int BD = 2;
        u32x4 Bq[BD + 1];
        auto lookup = [&](auto j_c) {
          constexpr int j = decltype(j_c)::value, i = j & 3;
          const u32x4& W = j < 4 ? W0 : W1;
          const unsigned d = __builtin_amdgcn_alignbyte(i < 3 ? W[i < 3 ? i + 1 : 0] : (j < 4 ? x0 : x1), W[i], dlt);
#pragma unroll
          for (int w = 0; w < 4; ++w)  // (byte 1 of the address: byte w of d; byte 0: 4 lane)
            Bq[j % (BD + 1)][w] = *(const lds_u32*)__builtin_amdgcn_perm(d, lane4, 0x0c0c0400u + ((unsigned)w << 8));
        };
        f32x4 C[NTOK];  // (a pair: one accumulator tile per window)
#pragma unroll
        for (int q = 0; q < NTOK; ++q) C[q] = f32x4{0.f, 0.f, 0.f, 0.f};
        lookup(IC<0>{});
        lookup(IC<1>{});
        auto stage = [&](auto j_c) {
          constexpr int j = decltype(j_c)::value, ci = NTOK == 1 ? 0 : j >> 2;
          __builtin_amdgcn_sched_barrier(0);
          if (j + BD < 8) lookup(IC<(j + BD < 8 ? j + BD : 0)>{});
          __builtin_amdgcn_sched_barrier(0);
          const u32x4 bq = Bq[j % (BD + 1)];
          const i32x8 B8 = {(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w, 0, 0, 0, 0};
          C[ci] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[j], B8, C[ci], 0 /* A: E4M3 */, 4 /* B: E2M1 */, 0, 0, 0, 0);
        };
        stage(IC<0>{}); stage(IC<1>{}); stage(IC<2>{}); stage(IC<3>{}); stage(IC<4>{}); stage(IC<5>{}); stage(IC<6>{}); stage(IC<7>{});
        __builtin_amdgcn_sched_barrier(0);
        const float sa = SDT == BP_F32 ? __uint_as_float(ra) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)ra) : __uint_as_float(ra << 16);
        const float sb = SDT == BP_F32 ? __uint_as_float(rbits) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)rbits) : __uint_as_float(rbits << 16);
        // the row's sum over its four lanes (one per quarter): row n ends up in every lane n + 16 q
#pragma unroll
        for (int tt = 0; tt < NTOK; ++tt) {
          float v;
          if (NTOK == 1) {
            v = sa * inv_a[0] * (C[0][0] + C[0][1] + C[0][2] * (1.f / 256.f)) + sb * inv_b[0] * C[0][3];
          } else {  // rows 4 kb + 2 tt + p of the two windows' tiles
            const f32x4 c0 = C[0], c1 = C[NTOK - 1];
            v = sa * inv_a[tt] * (tt ? c0[2] + c0[3] : c0[0] + c0[1]) + sb * inv_b[tt] * (tt ? c1[2] + c1[3] : c1[0] + c1[1]);
          }
          const auto h32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
          v = __uint_as_float(h32[0]) + __uint_as_float(h32[1]);
          const auto h16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
          v = __uint_as_float(h16[0]) + __uint_as_float(h16[1]);
          if (kb == 0) *(lds_u32*)(red + (unsigned)((((t % NB) * nchunks + c) * NTOK + tt) * 64 + 4 * r16)) = __float_as_uint(v);
        }
      };
      // Four token rows: instruction j multiplies piece j of the chunk (the lane's dword kb of it and the dword behind it,
      // for the realignment); accumulator tiles 0 .. 3 take instructions 0-2, 3, 4-5, 6-7. A lane of the result holds
      // slot kb / 2 of tokens 2 (kb % 2) and 2 (kb % 2) + 1: the sums of the slot's groups under their scales and the
      // tokens' inverse prescales, and the other slot's lane (kb ^ 2) has the rest of the row's sum.
      auto multiply4 = [&](int t) {
        const unsigned rb = gbase + (unsigned)((t % NB) * buf_bytes);
        const unsigned ra = SB == 4 ? *(const lds_u32*)(rb + rd_sa) : (unsigned)*(const lds_u16*)(rb + rd_sa);
        const unsigned rbits = SB == 4 ? *(const lds_u32*)(rb + rd_sb) : (unsigned)*(const lds_u16*)(rb + rd_sb);
        const unsigned rcb = SB == 4 ? *(const lds_u32*)(rb + rd_sc) : (unsigned)*(const lds_u16*)(rb + rd_sc);
        constexpr int BD = 2;
        u32x4 Bq[BD + 1];
        auto lookup = [&](auto j_c) {
          constexpr int j = decltype(j_c)::value;
          const unsigned cur = *(const lds_u32*)(rb + rd_w4 + 16 * j), nxt = *(const lds_u32*)(rb + rd_w4 + 16 * j + 4);
          const unsigned d = __builtin_amdgcn_alignbyte(nxt, cur, dlt);
#pragma unroll
          for (int w = 0; w < 4; ++w) Bq[j % (BD + 1)][w] = *(const lds_u32*)__builtin_amdgcn_perm(d, lane4, 0x0c0c0400u + ((unsigned)w << 8));
        };
        f32x4 C[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) C[q] = f32x4{0.f, 0.f, 0.f, 0.f};
        lookup(IC<0>{});
        lookup(IC<1>{});
        auto stage4 = [&](auto j_c) {
          constexpr int j = decltype(j_c)::value, ci = j < 3 ? 0 : j == 3 ? 1 : j < 6 ? 2 : 3;
          __builtin_amdgcn_sched_barrier(0);
          if (j + BD < 8) lookup(IC<(j + BD < 8 ? j + BD : 0)>{});
          __builtin_amdgcn_sched_barrier(0);
          const u32x4 bq = Bq[j % (BD + 1)];
          const i32x8 B8 = {(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w, 0, 0, 0, 0};
          C[ci] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A[j], B8, C[ci], 0 /* A: E4M3 */, 4 /* B: E2M1 */, 0, 0, 0, 0);
        };
        stage4(IC<0>{}); stage4(IC<1>{}); stage4(IC<2>{}); stage4(IC<3>{}); stage4(IC<4>{}); stage4(IC<5>{}); stage4(IC<6>{}); stage4(IC<7>{});
        __builtin_amdgcn_sched_barrier(0);
        auto widen = [&](unsigned r) { return SDT == BP_F32 ? __uint_as_float(r) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)r) : __uint_as_float(r << 16); };
        const float sa = widen(ra), sb = widen(rbits), sc = widen(rcb);
        const bool odd = (kb >> 1) != 0;  // the lane's slot
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          const float p0 = C[0][2 * t2] + C[0][2 * t2 + 1], p1 = C[1][2 * t2] + C[1][2 * t2 + 1];
          const float p2 = C[2][2 * t2] + C[2][2 * t2 + 1], p3 = C[3][2 * t2] + C[3][2 * t2 + 1];
          // slot 0: group 0 <- tile 0, group 2 <- tiles 1, 2, group 4 <- tile 3; slot 1: group 1 <- tiles 0, 1, group 3 <- tiles 2, 3
          const float qa = odd ? p0 + p1 : p0, qb = odd ? p2 + p3 : p1 + p2;
          float v = sa * inv_a[t2] * qa + sb * inv_b[t2] * qb + sc * inv_c[t2] * p3;
          const auto h32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
          v = __uint_as_float(h32[0]) + __uint_as_float(h32[1]);
          const int tt = 2 * (kb & 1) + t2;
          if (kb < 2) *(lds_u32*)(red + (unsigned)((((t % NB) * nchunks + c) * NTOK + tt) * 64 + 4 * r16)) = __float_as_uint(v);
        }
      };
      if (term > 0) __syncthreads();  // (the previous term's last tiles have been added)
      for (int i = 0; i < n_int; ++i) {
        __syncthreads();  // (the tiles TPB i .. TPB i + TPB - 1 are in their buffers)
#pragma unroll
        for (int u = 0; u < TPB; ++u) {
          if constexpr (M4) multiply4(TPB * i + u);
          else multiply(TPB * i + u);
        }
      }
      __syncthreads();
    }
    return;
  }

  // ---- loaders (and waves without a role, which only keep the barriers' count)
  __syncthreads();  // (the multipliers have their operand A)
  if constexpr (M4) {
    build_table();
    __syncthreads();
  }
  for (int term = 0; term < a.n_terms; ++term) {
    if (term > 0) setup_term(term);
    // The sums of the tile of iteration t, token tt by the group's loader tt % lpg: lane (row n, quarter q) adds chunks q,
    // q + 4, ... in that order, the row's four lanes are added in a fixed order too, and the row's entry of the output
    // stage takes one addition (this wave is the only one that touches its tokens' entries of its group between the
    // first barrier and the end).
    auto reduce = [&](int t, auto) {
      if (!loader) return;  // (uniform)
      const int64_t tile = tile_of(t);
#pragma unroll
      for (int tt = 0; tt < NTOK; ++tt) {
        if (tt % lpg != lidx) continue;  // (uniform)
        float v = 0.f;
#pragma unroll
        for (int q = 0; q < CW_WAVES / 4; ++q) {
          const int ch = 4 * q + kb;
          const unsigned at = red + (unsigned)((((t % NB) * nchunks + (ch < nchunks ? ch : 0)) * NTOK + tt) * 64 + 4 * r16);
          const float part = __uint_as_float(*(const lds_u32*)at);
          v += ch < nchunks ? part : 0.f;
        }
        const auto h32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(h32[0]) + __uint_as_float(h32[1]);
        const auto h16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(h16[0]) + __uint_as_float(h16[1]);
        if (lane < 16 && tile < tile_end && tt < ntok) {
          const unsigned at_out = stage + (unsigned)((((int)(tile - tile0) * NTOK + tt) * 16 + lane) * 4);
          *(lds_u32*)at_out = __float_as_uint(__uint_as_float(*(const lds_u32*)at_out) + (a.x_dtype == BP_I8 ? v * xsc[tt] : v));
        }
      }
    };
    // Two tiles are in flight per loader: the tile parked before a barrier was requested two tiles ago.
    static_assert(TPB == 1 || TPB == 2, "tiles per barrier");
    if (term > 0) __syncthreads();  // (the previous term's last tiles have been multiplied)
    if (term > 0) {
      request(0, IC<0>{});
      request(1, IC<1>{});
    }
    for (int t = 0; t < TPB * n_int; t += 2) {
      park(t, IC<0>{});
      request(t + 2, IC<0>{});
      if constexpr (TPB == 1) {
        __syncthreads();
        if (t > 0) reduce(t - 1, IC<1>{});  // (multiplied before this barrier)
        if (t + 1 >= n_int) break;  // (uniform)
      }
      park(t + 1, IC<1>{});
      request(t + 3, IC<1>{});
      __syncthreads();
      if constexpr (TPB == 1) {
        reduce(t, IC<0>{});
      } else {
        if (t > 0) {
          reduce(t - 2, IC<0>{});
          reduce(t - 1, IC<1>{});
        }
      }
    }
    __syncthreads();
    if constexpr (TPB == 2) reduce(TPB * n_int - 2, IC<0>{});
    if (TPB == 2 || (n_int & 1) == 0) reduce(TPB * n_int - 1, IC<1>{});
    else reduce(n_int - 1, IC<0>{});
  }
  // ---- the group's loaders write their tokens' outputs back: the entries a wave has added to itself (no barrier), four
  // tiles per wave store
  if (loader) {
    for (int t = kb; t < n_iter; t += 4) {
      const int64_t tile = tile_of(t);
#pragma unroll
      for (int tt = 0; tt < NTOK; ++tt) {
        if (tt % lpg == lidx && tile < tile_end && tt < ntok)
          a.out[(tok + tt) * a.N + tile * 16 + r16] = __uint_as_float(*(const lds_u32*)(stage + (unsigned)((((int)(tile - tile0) * NTOK + tt) * 16 + r16) * 4)));
      }
    }
  }
}

// Launch of the chunk-per-wave kernel, or BP_ERR_UNSUPPORTED (no message) where it does not apply: more than 15 chunks
// per row, scales that are not dword-aligned, an expert whose rows or scales exceed a buffer descriptor, tile buffers
// that do not fit, or a call too small for it (each workgroup builds the table and the token's tile before it streams).
template <int SDT, int NTOK>
int launch_cw(const GemmArgs& a, hipStream_t s, int64_t nchunks, int cus, int first_row) {
  const char force = tuning().tq1;
  if (force == 'r') return BP_ERR_UNSUPPORTED;
  for (int t = 0; t < a.n_terms; ++t)
    if (((uintptr_t)a.w_scale[t] & 3) != 0) return BP_ERR_UNSUPPORTED;
  constexpr int64_t SB = SDT == BP_F32 ? 4 : 2;
  if (a.N * a.Kp >= 0x7fffffe0 || a.N * a.G * SB >= 0x7fffffe0) return BP_ERR_UNSUPPORTED;
  const int64_t experts = a.E < a.T ? a.E : a.T, tiles = a.N / 16;
  if (force != 'c' && experts * tiles < 16 * (int64_t)cus) return BP_ERR_UNSUPPORTED;
  int64_t wpe = cus / experts;  // workgroups per expert: one workgroup per CU is resident
  wpe = wpe < 1 ? 1 : wpe > tiles ? tiles : wpe;
  int64_t per = (tiles + wpe - 1) / wpe;  // tiles per workgroup
  const int64_t buf = cw_buffer_bytes(a.Kp, a.G, SB);
  const int64_t nl = 4 * cw_colblks(a.Kp), ns = (16 * a.G * SB + 1023) / 1024;  // wave loads per tile: packed bytes, scales
  // A group: nchunks multipliers and its loaders, which take up to 8 wave loads of packed bytes each and one of the
  // scales. As many groups as fit the 16 waves, the tiles of a workgroup and LDS (two tiles per barrier if those fit too).
  auto loaders_of = [&](int g) { return (CW_WAVES - g * nchunks) / g; };
  // (a workgroup keeps its outputs in LDS: at most CW_STAGE_PER_THREAD per thread, 64 bytes per tile and token)
  const int64_t per_cap = CW_STAGE_PER_THREAD * CW_WAVES * 64 / (16 * NTOK);
  for (int64_t k = 2; per > per_cap; ++k) per = (tiles + k * wpe - 1) / (k * wpe);  // (twice, three times ... as many workgroups per expert: whole rounds of one workgroup per CU)
  auto lds_of = [&](int g, int tpb) {
    const int64_t stream = (int64_t)g * 2 * tpb * (buf + nchunks * 64 * NTOK), build = nchunks * NTOK * f4_chunk_bytes(NTOK);
    const int64_t mine = (per + g - 1) / g * g;  // tiles per workgroup with g groups
    if (NTOK == 4) return (CW_LUT_BYTES + stream > build ? CW_LUT_BYTES + stream : build) + mine * 64 * NTOK;  // (the tiles are built from LDS address 0)
    return (int64_t)CW_LUT_BYTES + (stream > build ? stream : build) + mine * 64 * NTOK;
  };
  auto fits = [&](int g, int tpb) {
    const int64_t l = loaders_of(g);
    return l >= 1 && l >= ns && (nl + l - 1) / l <= 8 && lds_of(g, tpb) <= F4_LDS_MAX;
  };
  int groups = (int)(CW_WAVES / (nchunks + 1));
  if (groups > per) groups = (int)per;
  while (groups > 1 && !fits(groups, 1)) --groups;
  if (groups < 1 || !fits(groups, 1)) return BP_ERR_UNSUPPORTED;
  const int tpb = fits(groups, 2) ? 2 : 1;
  const int64_t loaders = loaders_of(groups), lpw = (nl + loaders - 1) / loaders;
  per = (per + groups - 1) / groups * groups;
  if (per > per_cap) per = per_cap / groups * groups;
  // Measured against the kernel above (E x N x K from 64 x 4096 x 2048 to 256 x 2048 x 7168): ahead by 3 - 12 % with 10 or
  // more multipliers and 48 or more tiles per group, behind with fewer of either (7 multipliers at K = 4096; 21 tiles).
  if (force != 'c' && (groups * nchunks < 10 || per / groups < 48)) return BP_ERR_UNSUPPORTED;
  const dim3 grid((unsigned)((tiles + per - 1) / per), (unsigned)a.E, 1u);
  const size_t lds = (size_t)lds_of(groups, tpb);
  const char* const kname = NTOK == 1 ? "fp4_tq1_t1_cw" : NTOK == 2 ? "fp4_tq1_m2_cw" : "fp4_tq1_m4_cw";
  note_kernel(kname);
#define BP_CW_LAUNCH(L, P)                                                                                                                  \
  {                                                                                                                                         \
    if (const int rc = raise_lds_limit<k_tq1_gemv_cw<SDT, L, P, NTOK>>(F4_LDS_MAX)) return rc;                                              \
    hipLaunchKernelGGL((k_tq1_gemv_cw<SDT, L, P, NTOK>), grid, dim3(CW_WAVES * 64), lds, s, a, (int)nchunks, groups, (int)per, first_row); \
    return check_launch(kname);                                                                                                           \
  }
#define BP_CW_LPW(L)        \
  if (lpw == L) {           \
    if (tpb == 2) BP_CW_LAUNCH(L, 2) \
    BP_CW_LAUNCH(L, 1)      \
  }
  BP_CW_LPW(1) BP_CW_LPW(2) BP_CW_LPW(3) BP_CW_LPW(4) BP_CW_LPW(5) BP_CW_LPW(6) BP_CW_LPW(7) BP_CW_LPW(8)
#undef BP_CW_LPW
#undef BP_CW_LAUNCH
  return BP_ERR_UNSUPPORTED;
}

}  // namespace

int launch_tq1_gemv_cw(const GemmArgs& a, hipStream_t s, int ntok, int64_t nchunks, int cus, int first_row) {
  if (ntok == 4) {  // (2-byte scales)
    if (a.scale_dtype == BP_F16) return launch_cw<BP_F16, 4>(a, s, nchunks, cus, first_row);
    if (a.scale_dtype == BP_BF16) return launch_cw<BP_BF16, 4>(a, s, nchunks, cus, first_row);
    return BP_ERR_UNSUPPORTED;
  }
  if (ntok != 1 && ntok != 2) return BP_ERR_UNSUPPORTED;
  if (a.scale_dtype == BP_F16) return ntok == 1 ? launch_cw<BP_F16, 1>(a, s, nchunks, cus, first_row) : launch_cw<BP_F16, 2>(a, s, nchunks, cus, first_row);
  if (a.scale_dtype == BP_BF16) return ntok == 1 ? launch_cw<BP_BF16, 1>(a, s, nchunks, cus, first_row) : launch_cw<BP_BF16, 2>(a, s, nchunks, cus, first_row);
  if (a.scale_dtype == BP_F32) return ntok == 1 ? launch_cw<BP_F32, 1>(a, s, nchunks, cus, first_row) : launch_cw<BP_F32, 2>(a, s, nchunks, cus, first_row);
  return BP_ERR_UNSUPPORTED;
}

}  // namespace bp

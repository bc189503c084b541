// TQ1 decode GEMV (one token row per expert; small batches of up to 8 rows per expert and launch: NTOK below) on the
// block-float matrix instruction
// v_mfma_f32_16x16x128_f8f6f4, weights as fp4 (E2M1 holds -1, 0, +1 exactly), activations as fp8 (E4M3) pieces.
//
// Contract as everywhere (boilerplate/kernels/ternary_cuda.py:58-63): out[n] += sum_g scale[n, g] * sum_{k in g}
// x[k] * trit[n, k], float32 accumulation. What bounds a TQ1 GEMV on this chip is the work per packed byte: base-3
// digits have no bit fields, so a byte must go through a table, and a table of partial sums costs two LDS reads
// and ~10 vector operations per byte (bp_tq1_gemv.hip: a third of the HBM rate at best). Here a byte costs ONE
// conflict-free LDS read and two vector operations:
//
//  * The table maps a byte to its five digits as five fp4 codes in one dword (three more nibbles stay 0). A
//    lane's dword is used as is as a quarter of its operand B of the matrix instruction, so there is no unpacking.
//    The table is replicated once per LDS bank (entry v, copy c at v * 128 + 4 c; a lane reads copy lane % 32), so
//    no two lanes of a half-wave ever share a bank.
//  * K order inside a matrix instruction is free as long as both operands agree, so the bytes a lane loaded (16
//    consecutive bytes of its row per load, rows of a 16-row tile across lanes % 16, the four 16-byte quarters
//    of a 64-byte span across lanes / 16) are multiplied where they are: no transpose through LDS.
//  * The 16 rows of operand A are not tokens (there is one token) but (scale group, piece): a 128-byte chunk of a
//    row holds 640 digits = 5 scale groups, and an activation is split into 3 fp8 pieces (below), 15 rows in all.
//    Row (g, p) holds piece p of the activations of group g and zeros elsewhere, so one accumulator tile collects
//    the 5 group sums of a chunk separately although groups end in the middle of bytes, and the group scales
//    are applied once per chunk: total += scale[n, g] * (C[g, 0] + C[g, 1] + C[g, 2] / 256) / prescale[g].
//    Rows 4 g + p are the pieces of group g < 4 and rows 3, 7, 11 those of group 4, so a lane of the result (rows
//    4 kb + i) holds the three pieces of group kb and one piece of group 4.
//  * fp8 pieces: the activations of a 128-wide group are multiplied by a power of two that brings the group's
//    largest magnitude into [128, 256), then y = p0 + p1 + p2 / 256 with p0 = y rounded to E4M3 (4 significant
//    bits), p1 = the remainder rounded likewise, p2 = 256 x the second remainder, rounded (v_cvt_pk_fp8_f32: OCP
//    E4M3, round to nearest even, and v_cvt_f32_fp8 back; checked on gfx950). bf16 (8 significant bits) and int8
//    activations are exactly p0 + p1 down to 2^-9 of the group's largest magnitude, fp16 (11 bits) exactly the
//    three; below that a value keeps 4 more bits through p2, and what is dropped is less than 2^-20 of the group's
//    largest magnitude. Products fp8 x fp4 are exact and accumulate in float32. float32 activations (24 bits)
//    are left to the table kernel. A NaN or an infinity among a group's activations makes the token's outputs NaN
//    (the group's inverse prescale is NaN); the reference skips zero weights, so there only rows with a nonzero weight
//    at that k become non-finite.
//
// Operand A is read from an LDS tile built once per workgroup. It is stored compactly: per chunk, per matrix
// instruction j = 0..7 and per 16-byte half of an A lane's operand (= the 2 x 8 digit slots of two consecutive
// packed bytes) one block per piece with the digits outside the block's first group zeroed, a second block for
// each of the 4 byte pairs that straddle a group boundary (digits outside the second group zeroed), and a block
// of zeros. A lane (row (g, p)) reads the block of its piece if the byte pair lies in its group, else the zero
// block; which one is a per-lane offset computed once.
//
// Rows start at any byte (Kp = ceil(K / 5) is not a multiple of 4), loads are dword-aligned (a misaligned
// 16-byte load costs a quarter of the achievable HBM rate), and every row must present the same bytes to the
// shared operand A: a lane shifts its window by its row's misalignment with v_alignbyte, taking the dword that
// follows its 16 bytes from the lane that loaded it (ds_bpermute).
//
// Operand layout of the instruction with A = fp8 (8 VGPRs), B = fp4 (4 VGPRs), established by one-hot probing
// on gfx950: B lane (n = lane % 16, kb = lane / 16), VGPR w, nibble q is paired with A lane (m = lane % 16,
// kbA = 2 (kb % 2) + w / 2), VGPR 4 (kb / 2) + 2 (w % 2) + q / 4, byte q % 4; C lane (n, lg) holds rows 4 lg + i.
#include "bp_tq1_fp4.h"

namespace bp {
namespace {

// ABL (development): timing ablations - 1 no chunk loop, 2 no table reads, 3 no operand A reads, 4 no matrix instructions, 5 no byte extraction (and the loads are not waited for),
// 6 bytes extracted from registers that are not loaded (no loads at all), 7 = 2 + 3 + 4 (loads and byte extraction only),
// 8 = 7 without the byte extraction (loads and their realignment only)
//
// NTOK > 1: up to NTOK token rows per expert (small decode batches). Every token has its own operand A tile; the
// packed bytes and the table reads are shared. To fit 4 tiles beside the table, an activation is then split into
// TWO fp8 pieces (PC = 2: exact for bf16 / int8 values down to 2^-9 of their group's largest magnitude, at most
// 2^-17 of it dropped below), and one matrix instruction serves TWO tokens: the 64-byte window (half a chunk, 320
// digits) that instructions 0..3, and the one that instructions 4..7 multiply holds digits of only 3 groups
// (0, 1, 2 and 2, 3, 4), so a token needs 3 group slots x 2 pieces = 6 rows instead of 10 if each window has its
// own accumulator tile. Row 4 s + 2 t + p = piece p of token t (of the pair) in slot s; slot s is group s in the
// first window and group 3, 4, 2 (s = 0, 1, 2) in the second, so a lane of the result (rows 4 lg + i) holds both
// tokens' pieces of one group per window. 8 matrix instructions per chunk and token pair; with two pairs the ring
// of loads is two chunks (registers; the loads are not what a wave then waits for).
//
// SR (one token, 2-byte scales): scales by the round. A scale per row and group loaded where it is applied is a wave
// load per chunk that touches 16 memory lines for 8 bytes each: a third of the kernel's load instructions for 7 % of its
// bytes. Instead a wave loads, once per round of the ring (4 chunks = 20 groups = 40 bytes of a row's scales), 16 bytes
// per lane (quarters 0..2 of a row's four lanes cover 48 bytes), a round ahead and unconditionally - so the compiler's
// count of loads in flight stays exact - parks them in a private 1.25 KiB slot of LDS at the start of the round, and a
// chunk's two scales per lane are two 2-byte LDS reads.
// KS (one token, a call with few row tiles): the waves of a workgroup share one row tile and split its chunks - wave w
// takes chunks w cpw .. w cpw + cpw - 1 - and their partial sums are added through LDS in wave order. A call with 128
// row tiles then runs on 128 CUs for a sixth of the chunks each, where whole rows per wave keep 16 CUs busy.
template <int SDT, int WAVES, int ABL = 0, int NTOK = 1, int SR = 0, int KS = 0>
__global__ __launch_bounds__(WAVES * 64, KS ? 2 : 4) void k_tq1_gemv_fp4(GemmArgs a, int total_chunks, int first_chunk, int nchunks, int bpw /* row blocks per workgroup */, int first_row) {
  static_assert(!SR || (SDT != BP_F32 && F4_GR == 1), "scales by the round: one tile per wave, 2-byte scales (a round of 2 or 4 chunks is 20 or 40 bytes of a row's scales)");
  static_assert(!KS || (NTOK == 1 && F4_GR == 1 && ABL == 0), "chunks split over the waves: one token, one tile per workgroup");
  constexpr int THREADS = WAVES * 64, GR = F4_GR, RD = NTOK <= 2 ? F4_RD : 2, BD = F4_BD, AD = F4_AD, PAIRS = NTOK <= 2 ? F4_PAIRS : 0;
  static_assert(!PAIRS || RD % 2 == 0, "pairs of chunks need an even ring");
  static_assert(NTOK == 1 || (GR == 1 && AD == 0 && NTOK % 2 == 0), "several tokens: one tile per wave, one operand A buffer, token pairs");
  constexpr int NP = NTOK / 2;               // token pairs
  constexpr int PC = f4_pieces(NTOK);        // fp8 pieces per activation
  constexpr int F4_INV_OFF = F4Tile<PC>::INV_OFF, F4_CHUNK_BYTES = F4Tile<PC>::CHUNK_BYTES;
  constexpr int AT = F4_LUT_BYTES;           // the operand A tiles (one per token) start after the table
  constexpr int SB = SDT == BP_F32 ? 4 : 2;  // bytes per scale

  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, kb = lane >> 4;
  const int64_t e = blockIdx.y;
  const int64_t o0 = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  // A launch takes the expert's token rows first_row .. first_row + NTOK - 1 (one token: its first row); an expert with
  // more rows than that gets further launches, one without any in this range is done at once (uniform).
  const int64_t tok = o0 + (NTOK == 1 ? 0 : first_row);
  // (KS: the offsets are waited for behind the first loads of packed bytes, which do not depend on them)
  if (!KS && tok >= o1) return;
  const int ntok = o1 - tok < NTOK ? (int)(o1 - tok) : NTOK;
  const int npairs = (ntok + 1) >> 1;  // token pairs the expert has in this launch: the others' matrix instructions are left out
  float xsc[NTOK];  // int8 activations: the tokens' scales
#pragma unroll
  for (int tt = 0; tt < NTOK; ++tt) xsc[tt] = !KS && a.x_dtype == BP_I8 && tt < ntok ? a.x_scale[tok + tt] : 1.f;  // (KS: read behind the first loads, below)
  // the tiles of the NTOK tokens are interleaved chunk by chunk (a pair's tiles are a constant apart)
  auto tile_at = [](int tt, int c) { return AT + (c * NTOK + tt) * F4_CHUNK_BYTES; };
  const int gs = a.group == 256 ? 1 : 0;  // scale groups of 256: two 128-wide work groups share a scale

  // KS: the table and the token's tiles are built behind the first loads of packed bytes (in all_terms below), whose
  // latency then passes while the workgroup builds (such a call is mostly latencies in a row; the registers that the
  // loads in flight hold during the build are there with one workgroup per CU).
  constexpr bool LATE = KS != 0;
  if (!LATE) f4_build_table<THREADS>();
  // A launch covers the chunks first_chunk .. first_chunk + nchunks - 1 of every row (all of them unless the tokens'
  // tiles of all chunks do not fit in LDS: then the host launches once per segment of K, and the output takes the
  // segments' partial sums one launch after the other). Chunk c below is chunk cb + c of the rows.
  // (KS: this wave's chunks; a wave past the row's last chunk has none and only meets the others at the barriers)
  const int cpw = KS ? (nchunks + WAVES - 1) / WAVES : nchunks;
  const int cb = KS ? (wave * cpw < nchunks ? wave * cpw : nchunks) : NTOK == 1 ? 0 : first_chunk;
  const int nch = KS ? (nchunks - cb < cpw ? nchunks - cb : cpw) : nchunks;  // chunks this wave multiplies
  // The last bytes of a chunk are completed from the first dword of the chunk after it (rows start at any byte). At
  // the end of a row that dword meets activations that are 0; at the end of a segment it is needed, so the chunk
  // after a segment that is not the last one is loaded as well.
  // (Rows of whole chunks - Kp a multiple of 128 - at an address that is not a multiple of 4 end up to 3 bytes into the
  // chunk after their last one, with bytes that count: that chunk is loaded too; the term sets last_load below.)
  const int last_load_aligned = (NTOK > 1 || KS) && cb + nch < total_chunks ? nch : nch - 1;
  int last_load = last_load_aligned;

  if (!LATE) {
    f4_build_tiles<NTOK, WAVES>(a, tok, ntok, nchunks, KS ? 0 : cb, wave, lane);  // (KS: the tiles of all chunks, tile index = chunk)
    __syncthreads();
  }
  const int tb = KS ? cb : 0;  // tile index of the wave's chunk 0

  const unsigned lane_tok = PC == 2 ? (unsigned)(((r16 >> 1) & 1) * F4_CHUNK_BYTES) : 0u;  // the lane's token of a pair: its tile
  unsigned aoff[4];  // 16-byte block (index within the chunk's part of the tile) of instruction j, half hf: byte 2 (j % 2) + hf of aoff[j / 2]
  f4_block_offsets<PC>(r16, kb, aoff);
  // ---- this lane as a column of the result: rows 4 kb + i of C: pieces 0..2 of group kb, and piece kb of group 4
  const float f4th = kb == 3 ? 0.f : kb == 2 ? 1.f / 256.f : 1.f;
  const unsigned lane4 = (unsigned)(lane & 31) << 2;
  const unsigned next_lane4 = (unsigned)((lane + 16) & 63) << 2, last_lane4 = (unsigned)(48 + r16) << 2;

  // The tables serve `bpw` blocks of WAVES x GR x 16 rows, one after the other (the build is paid once per workgroup),
  // term by term: a term's blocks form one stream of chunks, and when the chunks of a row fill the ring a whole
  // number of times the refills run on into the next block, so the loads do not drain between blocks.
  bool chain = false;  // (set by the term)
  auto block_row = [&](int pass) -> int64_t {  // first row of this wave's tile(s) in block `pass`
    if (KS) return ((int64_t)blockIdx.x * bpw + pass) * (16 * GR);
    return (((int64_t)blockIdx.x * bpw + pass) * WAVES + wave) * (16 * GR);
  };
  auto block_row0 = [&](int pass) -> int64_t {  // ... or 0 (valid, not stored) past N
    const int64_t r = block_row(pass);
    return r < a.N ? r : 0;
  };
  // (the whole loop nest once per number of token pairs the expert has in this launch, chosen outside it: a branch
  // around the absent pairs' matrix instructions inside the chunk loop cost 18-43 spilled registers)
  auto all_terms = [&](auto npr_c) {
  constexpr int NPR = decltype(npr_c)::value;  // token pairs processed
  for (int term = 0; term < a.n_terms; ++term) {
    // the expert's rows as a buffer that ends with the tensor; dword-aligned base, per-lane row offset. A block
    // starts a multiple of 16 rows = of 4 bytes further on, so the misalignment is the same for all blocks.
    const unsigned char* wbeg = a.packed[term];
    const unsigned char* expert_rows = wbeg + e * a.N * a.Kp;
    const unsigned mis = (unsigned)((uintptr_t)expert_rows & 3);
    last_load = mis != 0 && a.Kp == 128 * (int64_t)total_chunks && cb + nch == total_chunks ? nch : last_load_aligned;
    chain = !KS && nchunks % RD == 0 && last_load == nchunks - 1;
    const __amdgpu_buffer_rsrc_t wrs = make_rsrc(expert_rows - mis, whole_dwords((wbeg + a.E * a.N * a.Kp) - (expert_rows - mis)));
    const unsigned ro = mis + (unsigned)r16 * (unsigned)a.Kp;
    const unsigned dlt = ro & 3u;  // the lane's window starts dlt bytes before its bytes of the row
    const unsigned voff = (ro & ~3u) + 16u * kb;
    const unsigned char* sbeg = (const unsigned char*)a.w_scale[term];
    const unsigned char* expert_scales = sbeg + e * a.N * a.G * SB;
    const unsigned smis = (unsigned)((uintptr_t)expert_scales & 3);
    const __amdgpu_buffer_rsrc_t srs = make_rsrc(expert_scales - smis, whole_dwords((sbeg + a.E * a.N * a.G * SB) - (expert_scales - smis)));
    const unsigned srow = smis + (unsigned)r16 * (unsigned)a.G * SB;
    u32x4 W[RD][GR][2];
    u32x2 SQ[GR];  // the scales of one chunk: refilled for the next chunk as soon as they have been applied
    // (SR) the wave's scale slot behind the tiles: [16 rows][80 bytes], 48 of them the scales of the round's 20 groups
    const unsigned sr_at = (unsigned)(AT + nchunks * NTOK * F4_CHUNK_BYTES + wave * F4_SCALE_SLOT + r16 * 80);
    u32x4 SN = {0u, 0u, 0u, 0u};  // (SR) the next round's scales of this lane's row: 16 bytes at 16 kb

  for (int pass = 0; pass < bpw; ++pass) {
    const int64_t n0 = block_row0(pass), n0_next = pass + 1 < bpw ? block_row0(pass + 1) : n0;
    const bool wave_live = block_row(pass) < a.N;
    float total[NTOK > 1 ? NTOK : GR];  // per token (this lane's two groups of every chunk), or (one token) per row tile
    // The outputs this block is added to are requested now and used when the block ends: read where they are added, the
    // load would be the youngest one in flight and the wait for it would drain the ring once per block. (Device scope:
    // with stacked terms the value may be one this wave stored a term ago.)
    // (up to 4 tokens; beyond, the registers are not there)
    constexpr bool EARLY = NTOK <= 4;
    float before[NTOK > 1 ? NTOK : GR];
#pragma unroll
    for (int s = 0; s < (NTOK > 1 ? NTOK : GR); ++s) {
      total[s] = 0.f;
      const int tile = NTOK > 1 ? 0 : s, tt = NTOK > 1 ? s : 0;
      before[s] = 0.f;
      if (EARLY && kb == 0 && wave_live && n0 + 16 * tile < a.N && tt < ntok && (!KS || wave == 0))
        before[s] = __hip_atomic_load(a.out + (tok + tt) * a.N + n0 + 16 * tile + r16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // chunk c of this block, or (c >= nchunks, chained) chunk c - nchunks of the next one: row offset (scalar) and chunk
    auto target = [&](int c, int64_t& row0, int& cc) {
      const bool over = chain && c >= nch && pass + 1 < bpw;
      row0 = over ? n0_next : n0;
      cc = over ? c - nch : (c < last_load ? c : last_load);
    };

    // RD chunks in registers per tile; a chunk's registers are refilled (RD chunks on) as soon as its last byte has
    // gone into a table read.
    auto fetch_w = [&](int c, int slot, int h) {
      int64_t row0;
      int cc;
      target(c, row0, cc);
#pragma unroll
      for (int s = 0; s < GR; ++s) {
        const int64_t row = row0 + 16 * s < a.N ? row0 + 16 * s : row0;  // a tile past N repeats tile 0 and is not stored
        W[slot][s][h] = buf_load16(wrs, voff, (unsigned)(row * a.Kp) + 128u * (unsigned)(cb + cc) + 64u * h);
      }
    };
    // (several tokens: the lane's group of the first window and the one of the second: lg and 3, 4, 2, 2 for lg = 0..3;
    // the lanes lg = 3 hold unused rows: their accumulators are 0)
    const int g_w0 = kb < 3 ? kb : 2, g_w1 = kb == 0 ? 3 : kb == 1 ? 4 : 2;
    auto fetch_s = [&](int c) {  // 8 bytes from the dword that holds the scale of group kb of chunk c
      int64_t row0;
      int cc;
      target(c, row0, cc);
      if (PC == 2) {  // the two dwords that hold the scales of the lane's two groups
        const unsigned at0 = (srow + SB * (unsigned)((5 * (cb + cc) + g_w0) >> gs)) & ~3u, at1 = (srow + SB * (unsigned)((5 * (cb + cc) + g_w1) >> gs)) & ~3u;
        const unsigned wo = (unsigned)(row0 * a.G * SB);
        SQ[0].x = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(srs, (int)at0, (int)wo, 0);
        SQ[0].y = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(srs, (int)at1, (int)wo, 0);
        return;
      }
      const unsigned at = (srow + SB * (unsigned)((5 * (cb + cc) + kb) >> gs)) & ~3u;
#pragma unroll
      for (int s = 0; s < GR; ++s) {
        const int64_t row = row0 + 16 * s < a.N ? row0 + 16 * s : row0;
        SQ[s] = f4_load8(srs, at, (unsigned)(row * a.G * SB));
      }
    };
    auto fetch_round = [&](int c) {  // (SR) the scales of the round that starts with chunk c (a multiple of 4; past the block: of the next one)
      int64_t row0;
      int cc;
      target(c, row0, cc);
      SN = buf_load16(srs, srow + 16u * kb, (unsigned)(row0 * a.G * SB) + ((SB * (unsigned)((5 * (cb + cc)) >> gs)) & ~3u));
    };
    // byte offset, within the parked window of its round, of the scale of group g of chunk c
    auto parked_at = [&](int c, int g) {
      // (one token: rounds of 4 chunks from chunk 0, so a round starts 20 groups = a whole number of dwords into the row)
      if (NTOK == 1 && !KS) return SB * (unsigned)((5 * (c & (RD - 1)) + g) >> gs);
      const unsigned first = (SB * (unsigned)((5 * (cb + (c & ~(RD - 1)))) >> gs)) & ~3u;
      return SB * (unsigned)((5 * (cb + c) + g) >> gs) - first;
    };
    auto park_round = [&]() { *(lds_u32x4*)(sr_at + 16 * kb) = SN; };
    // (chunk slots and pipeline stages are compile-time constants: every register array below is indexed statically)
    auto step = [&](int c, auto cur_c) {
      constexpr int cur = decltype(cur_c)::value, nxt = (cur + 1) % RD;
      constexpr int NC = NTOK > 1 ? NTOK : GR;  // accumulator tiles: per token pair and window, or (one token) one per row tile
      f32x4 C[NC];
#pragma unroll
      for (int s = 0; s < NC; ++s) C[s] = f32x4{0.f, 0.f, 0.f, 0.f};
      const unsigned cbase = (unsigned)tile_at(0, tb + c);
      // packed bytes of (instruction j, tile s) = dword j % 4 of the lane's window j / 4, shifted to the row's alignment;
      // the dword after a window is the first one of the next quarter's window (for the last quarter: of the first
      // quarter's next window, which for the second window is the next chunk's)
      unsigned w4[GR], last[GR];  // (last: the last dword of the second window, kept while its registers are refilled)
      auto bytes_of = [&](int j, int s) -> unsigned {
        const int h = j >> 2, i = j & 3;
        if (ABL == 5) return 0u;
        if (ABL == 6) return __builtin_amdgcn_alignbyte(aoff[(j + 1) & 3], aoff[j & 3] + j, dlt);  // same arithmetic, nothing loaded
        if (j == 7) return __builtin_amdgcn_alignbyte(w4[s], last[s], dlt);
        return __builtin_amdgcn_alignbyte(i < 3 ? W[cur][s][h][i < 3 ? i + 1 : 0] : w4[s], W[cur][s][h][i], dlt);
      };
      auto table = [&](unsigned d, u32x4& B) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const unsigned at = ABL == 5 ? (unsigned)(w << 7) | lane4 : ABL == 8 ? d : (((d >> (8 * w)) & 0xffu) << 7) | lane4;
          B[w] = ABL == 2 || ABL == 7 || ABL == 8 ? at : *(const lds_u32*)at;
        }
      };
      auto a_read = [&](int j, u32x4& lo, u32x4& hi) {  // (one token)
        if (ABL == 3 || ABL == 7 || ABL == 8) { lo = u32x4{cbase, dlt, lane4, cbase}; hi = lo; return; }
        lo = *(const lds_u32x4*)((((aoff[j >> 1] >> (16 * (j & 1))) & 0xffu) << 4) + cbase);
        hi = *(const lds_u32x4*)((((aoff[j >> 1] >> (16 * (j & 1) + 8)) & 0xffu) << 4) + cbase);
      };
      // software pipeline over the 16 (instruction, tile) pairs t = 2 j + s: table reads BD pairs ahead, operand A one
      // instruction ahead if AD; the scheduling barriers keep the compiler from sinking the reads back to their uses
      constexpr int NT = 8 * GR;  // (instruction, tile) pairs of a chunk
      u32x4 Bq[BD + 1];
      u32x4 Alo[AD + 1], Ahi[AD + 1];
      auto lookup = [&](auto p_c) {  // table reads of pair p
        constexpr int p = decltype(p_c)::value, j = p / GR, s = p % GR;
        if (j == 3)  // the dword after the first window: the first one of the next quarter's first window, or of the own second window
          w4[s] = (unsigned)__builtin_amdgcn_ds_bpermute((int)next_lane4, (int)(kb == 0 ? W[cur][s][1].x : W[cur][s][0].x));
        if (p == 7 * GR) {
          // The dword after the second window comes from the next quarter's second window, for the last quarter
          // from the next chunk. What the last instruction still needs of this chunk is set aside, the chunk's
          // registers are refilled (RD chunks on), and only then is the next chunk's first dword waited for: the
          // wave never waits with fewer than RD - 1 chunks in flight behind the one it waits for.
          unsigned same[GR];
#pragma unroll
          for (int q = 0; q < GR; ++q) {
            // (a copy the compiler cannot merge with its source: kept in the same register, it would make the refill
            // below load into other registers and copy them at the end of the loop - after waiting for the load)
            asm volatile("v_mov_b32 %0, %1" : "=v"(last[q]) : "v"(W[cur][q][1].w));
            same[q] = (unsigned)__builtin_amdgcn_ds_bpermute((int)next_lane4, (int)W[cur][q][1].x);
          }
          // Both windows together (the two loads of a row's 128 bytes then meet in the L1), and with PAIRS two
          // chunks together, after the second one of a pair has been consumed: 256 consecutive bytes of a row per
          // visit, so the 128-byte line that two chunks share is fetched once.
          if (!PAIRS) {
            fetch_w(c + RD, cur, 0);
            fetch_w(c + RD, cur, 1);
          } else if (cur & 1) {
            fetch_w(c + RD - 1, cur - 1, 0);
            fetch_w(c + RD - 1, cur - 1, 1);
            fetch_w(c + RD, cur, 0);
            fetch_w(c + RD, cur, 1);
          }
#pragma unroll
          for (int q = 0; q < GR; ++q) {
            const unsigned far = (unsigned)__builtin_amdgcn_ds_bpermute((int)next_lane4, (int)W[nxt][q][0].x);
            w4[q] = kb == 3 ? far : same[q];
          }
        }
        table(bytes_of(j, s), Bq[p % (BD + 1)]);
      };
      if (NTOK == 1) a_read(0, Alo[0], Ahi[0]);
      lookup(IC<0>{});
      if (BD > 1) lookup(IC<BD - 1>{});
      static_assert(BD <= 2 && GR <= 2 && RD <= 4, "the stage list below covers 16 pairs, the chunk loop 4 slots");
      auto stage = [&](auto t_c) {
        constexpr int t = decltype(t_c)::value, j = t / GR, s = t % GR;
        if (t + BD < NT) lookup(IC<(t + BD < NT ? t + BD : 0)>{});
        if (AD && s == 0 && j + 1 < 8) a_read(j + 1, Alo[(j + 1) & AD], Ahi[(j + 1) & AD]);

        const u32x4 bq = Bq[t % (BD + 1)];
        const i32x8 B = {(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w, 0, 0, 0, 0};
        if (NTOK > 1) {
          // The same packed bytes against every token pair's operand A, one pair at a time (the scheduling barriers
          // keep the compiler from reading all the operands first: 8 registers each). Tiles of tokens the expert does
          // not have hold whatever LDS held; their rows of the accumulators are not used.
          unsigned ao = aoff[j >> 1];
          // (the block offsets are extracted anew at every use: left visible, the compiler hoists the 16 addresses of
          // a lane out of the chunk loop, and they do not fit its registers)
          asm volatile("; packed block offsets" : "+v"(ao));
          const unsigned lo_at = (((ao >> (16 * (j & 1))) & 0xffu) << 4) + cbase + lane_tok;
          const unsigned hi_at = (((ao >> (16 * (j & 1) + 8)) & 0xffu) << 4) + cbase + lane_tok;
#pragma unroll
          for (int pr = 0; pr < NPR; ++pr) {
            __builtin_amdgcn_sched_barrier(0);
            const u32x4 alo = *(const lds_u32x4*)(lo_at + 2 * pr * F4_CHUNK_BYTES), ahi = *(const lds_u32x4*)(hi_at + 2 * pr * F4_CHUNK_BYTES);
            const i32x8 A = {(int)alo.x, (int)alo.y, (int)alo.z, (int)alo.w, (int)ahi.x, (int)ahi.y, (int)ahi.z, (int)ahi.w};
            constexpr int ci = j >> 2;  // the window's accumulator tile
            C[2 * pr + ci] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, C[2 * pr + ci], 0 /* A: E4M3 */, 4 /* B: E2M1 */, 0, 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          return;
        }
        __builtin_amdgcn_sched_barrier(0);
        const u32x4 alo = Alo[j & AD], ahi = Ahi[j & AD];
        const i32x8 A = {(int)alo.x, (int)alo.y, (int)alo.z, (int)alo.w, (int)ahi.x, (int)ahi.y, (int)ahi.z, (int)ahi.w};
        if (ABL == 4 || ABL == 7 || ABL == 8) asm volatile("; operands stay live" ::"v"(bq), "v"(alo), "v"(ahi));
        else C[s] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(A, B, C[s], 0 /* A: E4M3 */, 4 /* B: E2M1 */, 0, 0, 0, 0);
        if (!AD && s == GR - 1 && j + 1 < 8) a_read(j + 1, Alo[0], Ahi[0]);  // every tile has issued with this operand
        __builtin_amdgcn_sched_barrier(0);
      };
#define BP_F4_STAGE(T) if (T < NT) stage(IC<(T < NT ? T : 0)>{})
      BP_F4_STAGE(0); BP_F4_STAGE(1); BP_F4_STAGE(2); BP_F4_STAGE(3); BP_F4_STAGE(4); BP_F4_STAGE(5); BP_F4_STAGE(6); BP_F4_STAGE(7);
      BP_F4_STAGE(8); BP_F4_STAGE(9); BP_F4_STAGE(10); BP_F4_STAGE(11); BP_F4_STAGE(12); BP_F4_STAGE(13); BP_F4_STAGE(14); BP_F4_STAGE(15);
#undef BP_F4_STAGE
      // the chunk's 5 group sums under their scales. Three pieces: this lane holds group kb (3 pieces) and a piece of
      // group 4, whose scale sits next to that of group 3 in the lanes kb = 3. Several tokens: one group per window.
      const int g_first = PC == 3 ? kb : g_w0;
      const unsigned ia = (unsigned)((5 * (cb + c) + g_first) >> gs), ib = (unsigned)((5 * (cb + c) + (PC == 3 ? g_first + 1 : g_w1)) >> gs);
      if constexpr (SR != 0) {
        // the lane's two scales of the chunk from the round's parked window: group kb and group 4 (one token), or the
        // groups of its two windows (several tokens)
        const unsigned ra = *(const lds_u16*)(sr_at + parked_at(c, g_first));
        const unsigned rb = *(const lds_u16*)(sr_at + parked_at(c, PC == 3 ? 4 : g_w1));
        const float sa = SDT == BP_F16 ? f16_bits_to_f32((uint16_t)ra) : __uint_as_float(ra << 16);
        const float sb = SDT == BP_F16 ? f16_bits_to_f32((uint16_t)rb) : __uint_as_float(rb << 16);
        if (PC == 3) {
          const float inv_a = __uint_as_float(*(const lds_u32*)(cbase + F4_INV_OFF + 4 * kb));
          const float inv_4 = __uint_as_float(*(const lds_u32*)(cbase + F4_INV_OFF + 16)) * f4th;
          total[0] += sa * inv_a * (C[0][0] + C[0][1] + C[0][2] * (1.f / 256.f)) + sb * inv_4 * C[0][3];
        } else {
#pragma unroll
          for (int tt = 0; tt < 2 * NPR; ++tt) {  // rows 4 lg + 2 (tt % 2) + p of the pair's two tiles
            const unsigned ivb = cbase + (unsigned)(tt * F4_CHUNK_BYTES) + F4_INV_OFF;
            const float inv_a = __uint_as_float(*(const lds_u32*)(ivb + 4 * g_w0)), inv_b = __uint_as_float(*(const lds_u32*)(ivb + 4 * g_w1));
            const f32x4 c0 = C[2 * (tt >> 1)], c1 = C[2 * (tt >> 1) + 1];
            const float s0 = (tt & 1) ? c0[2] + c0[3] : c0[0] + c0[1], s1 = (tt & 1) ? c1[2] + c1[3] : c1[0] + c1[1];
            total[tt] += sa * inv_a * s0 + sb * inv_b * s1;
          }
        }
        return;
      }
#pragma unroll
      for (int s = 0; s < GR; ++s) {
        unsigned ra, rb;  // the scale of group g_first, and the one after it (bits as stored)
        if (SDT == BP_F32) {
          ra = SQ[s].x;
          rb = ib == ia ? ra : SQ[s].y;
        } else if (PC == 2) {
          ra = (SQ[s].x >> (8u * ((srow + SB * ia) & 3u))) & 0xffffu;
          rb = (SQ[s].y >> (8u * ((srow + SB * ib) & 3u))) & 0xffffu;
        } else {
          const unsigned v = __builtin_amdgcn_alignbyte(SQ[s].y, SQ[s].x, (srow + SB * ia) & 3u);
          ra = v & 0xffffu;
          rb = ib == ia ? ra : v >> 16;
        }
        const float sa = SDT == BP_F32 ? __uint_as_float(ra) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)ra) : __uint_as_float(ra << 16);
        if (PC == 3) {
          const float inv_a = __uint_as_float(*(const lds_u32*)(cbase + F4_INV_OFF + 4 * kb));
          const float inv_4 = __uint_as_float(*(const lds_u32*)(cbase + F4_INV_OFF + 16)) * f4th;
          const unsigned r4 = (unsigned)__builtin_amdgcn_ds_bpermute((int)last_lane4, (int)rb);
          const float s4 = SDT == BP_F32 ? __uint_as_float(r4) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)r4) : __uint_as_float(r4 << 16);
          total[s] += sa * inv_a * (C[s][0] + C[s][1] + C[s][2] * (1.f / 256.f)) + s4 * inv_4 * C[s][3];
        } else {  // (one row tile per wave: s == 0)
          const float sb = SDT == BP_F32 ? __uint_as_float(rb) : SDT == BP_F16 ? f16_bits_to_f32((uint16_t)rb) : __uint_as_float(rb << 16);
#pragma unroll
          for (int tt = 0; tt < 2 * NPR; ++tt) {  // rows 4 lg + 2 (tt % 2) + p of the pair's two tiles
            const unsigned ivb = cbase + (unsigned)(tt * F4_CHUNK_BYTES) + F4_INV_OFF;
            const float inv_a = __uint_as_float(*(const lds_u32*)(ivb + 4 * g_w0)), inv_b = __uint_as_float(*(const lds_u32*)(ivb + 4 * g_w1));
            const f32x4 c0 = C[2 * (tt >> 1)], c1 = C[2 * (tt >> 1) + 1];
            const float s0 = (tt & 1) ? c0[2] + c0[3] : c0[0] + c0[1], s1 = (tt & 1) ? c1[2] + c1[3] : c1[0] + c1[1];
            total[tt] += sa * inv_a * s0 + sb * inv_b * s1;
          }
        }
      }
      fetch_s(c + 1);
    };

    // The first loads (of a term, or of every block if the blocks are not chained), in the order of use and with the
    // scales last: the waits at the head of the loop are counted along this path too, and here as there the
    // loads of later chunks and of the scales are the ones in flight behind the chunk that is needed.
    if (pass == 0 || !chain) {
      // (SR: the first round's scales are requested before the ring's loads, as in the loop - where a round's refills lie
      // between a round's scales and the wait for them - so that the wait at the head of the loop counts those loads on
      // this path too and does not drain the ring)
      if (SR) fetch_round(0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < RD; ++u) {
        fetch_w(u, u, 0);
        fetch_w(u, u, 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (LATE && term == 0 && pass == 0) {  // (uniform)
        if (tok >= o1) return;  // (uniform for the workgroup and before its first barrier: this ends the kernel - all_terms is its last statement)
        if (a.x_dtype == BP_I8) xsc[0] = a.x_scale[tok];
        f4_build_table<THREADS>();
        f4_build_tiles<NTOK, WAVES>(a, tok, ntok, nchunks, KS ? 0 : cb, wave, lane);
        __syncthreads();
      }
      __builtin_amdgcn_sched_barrier(0);
      if (SR) park_round();
      else fetch_s(0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // RD chunks per iteration with no way around any of them: the compiler counts the loads in flight along every
    // path into the head of the loop, and a path on which fewer are in flight would make every iteration wait
    const int full_end = ABL == 1 ? 0 : nch - nch % RD;
    for (int c0 = 0; c0 < full_end; c0 += RD) {
      // (SR) the next round's scales are requested at the head of a round and parked in LDS at its end, after the
      // round's last scale has been read: the round's 8 refills of the ring lie between, in straight-line code
      if (SR) fetch_round(c0 + RD);
      step(c0, IC<0>{});
      step(c0 + 1, IC<1 % RD>{});
      if (RD > 2) step(c0 + 2, IC<2 % RD>{});
      if (RD > 3) step(c0 + 3, IC<3 % RD>{});
      if (SR) park_round();
    }
    if (ABL != 1 && nch - full_end > 0) step(full_end, IC<0>{});  // uniform
    if (ABL != 1 && nch - full_end > 1) step(full_end + 1, IC<1 % RD>{});
    if (ABL != 1 && nch - full_end > 2) step(full_end + 2, IC<2 % RD>{});
  // ---- the four quarter lanes of a row hold its partial sums (of this term: the output is added to)
#pragma unroll
  for (int s = 0; s < (NTOK > 1 ? NTOK : GR); ++s) {
    float t = total[s];
    t += __shfl_xor(t, 16);
    t += __shfl_xor(t, 32);
    const int tile = NTOK > 1 ? 0 : s, tt = NTOK > 1 ? s : 0;
    if constexpr (KS != 0) {  // the waves' partial sums of the tile's 16 rows, added in wave order by wave 0
      const unsigned red = (unsigned)(AT + nchunks * NTOK * F4_CHUNK_BYTES + (SR ? WAVES * F4_SCALE_SLOT : 0));
      if (kb == 0) *(lds_u32*)(red + (unsigned)((wave * 16 + r16) * 4)) = __float_as_uint(t);
      __syncthreads();
      if (wave == 0) {
        t = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) t += __uint_as_float(*(const lds_u32*)(red + (unsigned)((w * 16 + r16) * 4)));
      }
      __syncthreads();  // (the next term writes the same slots)
      if (wave != 0) continue;
    }
    if (kb == 0 && wave_live && n0 + 16 * tile < a.N && tt < ntok) {
      float* o = a.out + (tok + tt) * a.N + n0 + 16 * tile + r16;
      const float was = EARLY ? before[s] : __hip_atomic_load(o, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *o = was + (a.x_dtype == BP_I8 ? t * xsc[tt] : t);
    }
  }
  }  // pass
  }  // term
  };
  if (NP >= 2 && npairs == 1) all_terms(IC<1>{});
  else if (NP >= 3 && npairs == 2) all_terms(IC<(NP >= 3 ? 2 : NP)>{});
  else if (NP >= 4 && npairs == 3) all_terms(IC<(NP >= 4 ? 3 : NP)>{});
  else all_terms(IC<NP>{});
}
template <int SDT, int WAVES, int ABL = 0, int NTOK = 1, int SR = 0, int KS = 0>
int launch_f4_k(const GemmArgs& a, hipStream_t s, const char* name, int nchunks, size_t lds, int seg_chunks = 0 /* chunks per launch (0: all) */, int first_row = 0) {
  if (const int rc = raise_lds_limit<k_tq1_gemv_fp4<SDT, WAVES, ABL, NTOK, SR, KS>>(F4_LDS_MAX)) return rc;
  if (SR) lds += (size_t)WAVES * F4_SCALE_SLOT;
  if (KS) lds += (size_t)WAVES * 64;  // the waves' partial sums
  const int cus = f4_cus();
  // Every workgroup builds the tables of its expert's token, so a workgroup takes as many row blocks as still leaves
  // every CU its full set of resident workgroups (16 waves): all workgroups resident at once, one build each.
  const int64_t rows_per_block = (int64_t)(KS ? 1 : WAVES) * 16 * F4_GR;
  const int64_t blocks = (a.N + rows_per_block - 1) / rows_per_block;  // per expert
  const int64_t resident = (int64_t)cus * (16 / WAVES);
  const int64_t experts = a.E < a.T ? a.E : a.T;  // (an expert without a token returns at once)
  int64_t bpw = blocks * experts / resident;
  bpw = bpw < 1 || KS ? 1 : bpw > blocks ? blocks : bpw;
  const dim3 grid((unsigned)((blocks + bpw - 1) / bpw), (unsigned)a.E, 1u);
  note_kernel(name);
  const int per = seg_chunks > 0 ? seg_chunks : nchunks;
  for (int cb = 0; cb < nchunks; cb += per) {
    hipLaunchKernelGGL((k_tq1_gemv_fp4<SDT, WAVES, ABL, NTOK, SR, KS>), grid, dim3(WAVES * 64), lds, s, a, nchunks, cb, nchunks - cb < per ? nchunks - cb : per, (int)bpw, first_row);
    const int rc = check_launch(name);
    if (rc != BP_OK) return rc;
  }
  return BP_OK;
}

template <int SDT, int NTOK>
int launch_f4(const GemmArgs& a, hipStream_t s, int first_row = 0) {
  const int64_t nchunks = (a.K + 639) / 640;
  // several tokens: K in as many equal segments as make the tokens' tiles of one segment fit beside the table
  const int64_t fit = (F4_LDS_MAX - F4_LUT_BYTES) / (NTOK * f4_chunk_bytes(NTOK));
  const int64_t nseg = NTOK == 1 ? 1 : (nchunks + fit - 1) / fit, seg = (nchunks + nseg - 1) / nseg;
  const size_t lds = (size_t)(F4_LUT_BYTES + NTOK * seg * f4_chunk_bytes(NTOK));
  if (lds > (size_t)F4_LDS_MAX || nseg > 4) return BP_ERR_UNSUPPORTED;
  const int cus = f4_cus();
  const int64_t experts = a.E < a.T ? a.E : a.T;
  // 2-byte scales go by the round through LDS where the slots fit behind the tiles and a row's scales start dword-aligned
  constexpr int SRV = SDT != BP_F32 && NTOK <= 4 ? 1 : 0;
  const bool sr_ok = SRV && (a.G * 2) % 4 == 0;
  if constexpr (NTOK == 2) {  // (a pair of rows per expert in a large call: the rows through LDS tile by tile)
    if (nseg == 1) {
      const int rc = launch_tq1_gemv_cw(a, s, 2, nchunks, cus, first_row);
      if (rc != BP_ERR_UNSUPPORTED) return rc;
    }
  }
  if constexpr (NTOK == 4) {  // (four rows per expert in a large call: the same, a matrix instruction per 16-byte piece)
    if (tuning().tq1 != 'r') {
      const int rc = launch_tq1_gemv_cw(a, s, 4, nchunks, cus, first_row);
      if (rc != BP_ERR_UNSUPPORTED) return rc;
    }
  }
  if (NTOK > 1) {
    const bool wide = lds > (size_t)F4_LDS_MAX / 2 || ((a.N + 255) / 256) * experts >= 4 * (int64_t)cus;
    const char* name8 = NTOK == 2 ? "fp4_tq1_m2_w8" : NTOK == 4 ? "fp4_tq1_m4_w8" : NTOK == 6 ? "fp4_tq1_m6_w8" : "fp4_tq1_m8_w8";
    const char* name16 = NTOK == 2 ? "fp4_tq1_m2_w16" : NTOK == 4 ? "fp4_tq1_m4_w16" : NTOK == 6 ? "fp4_tq1_m6_w16" : "fp4_tq1_m8_w16";
    if (!wide) {
      if (sr_ok && lds + 8 * F4_SCALE_SLOT <= (size_t)F4_LDS_MAX) return launch_f4_k<SDT, 8, 0, NTOK, SRV>(a, s, name8, (int)nchunks, lds, (int)seg, first_row);
      return launch_f4_k<SDT, 8, 0, NTOK>(a, s, name8, (int)nchunks, lds, (int)seg, first_row);
    }
    if (sr_ok && lds + 16 * F4_SCALE_SLOT <= (size_t)F4_LDS_MAX) return launch_f4_k<SDT, 16, 0, NTOK, SRV>(a, s, name16, (int)nchunks, lds, (int)seg, first_row);
    return launch_f4_k<SDT, 16, 0, NTOK>(a, s, name16, (int)nchunks, lds, (int)seg, first_row);
  }
  {
    const int rc = launch_tq1_gemv_cw(a, s, 1, nchunks, cus, 0);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
#ifdef BP_DEV_ABLATIONS  // timing ablations (results are wrong): development builds only
  if (const char* t = getenv("BP_TUNE_F4ABL")) {
    if (SDT == BP_F16 && atoi(t) == 1) return launch_f4_k<BP_F16, 8, 1>(a, s, "abl1_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 2) return launch_f4_k<BP_F16, 8, 2>(a, s, "abl2_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 3) return launch_f4_k<BP_F16, 8, 3>(a, s, "abl3_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 4) return launch_f4_k<BP_F16, 8, 4>(a, s, "abl4_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 5) return launch_f4_k<BP_F16, 8, 5>(a, s, "abl5_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 6) return launch_f4_k<BP_F16, 8, 6>(a, s, "abl6_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 7) return launch_f4_k<BP_F16, 8, 7>(a, s, "abl7_fp4", (int)nchunks, lds);
    if (SDT == BP_F16 && atoi(t) == 8) return launch_f4_k<BP_F16, 8, 8>(a, s, "abl8_fp4", (int)nchunks, lds);
  }
#endif
  // Two workgroups of 8 waves per CU when their tiles fit side by side and the call is small; one of 16 waves when
  // there are row blocks enough for every CU anyway (the tables are then built once per CU instead of twice).
  bool wide = lds > (size_t)F4_LDS_MAX / 2 || ((a.N + 255) / 256) * experts >= 4 * (int64_t)cus;
  if (tuning().f4w) wide = lds > (size_t)F4_LDS_MAX / 2 || tuning().f4w == 16;  // (development)
  constexpr int SR = SRV;
  if (!wide) {
    if constexpr (SDT != BP_F32) {
      // A call with few row tiles (one linear of a decode step) is mostly set-up, table and token tile, which every
      // workgroup repeats: workgroups of 4 waves put the tiles on twice as many CUs (measured, N = 2048, K = 7168, one
      // expert: 16.7 us per call against 17.3; workgroups of 2 waves 19.8, of 1 wave 27.3: fewer threads build longer).
      const int64_t tiles = ((a.N + 15) / 16) * experts;
      // ... and with no more row tiles than CUs, a tile per workgroup with its chunks split over the 8 waves
      const bool split = tuning().f4w ? tuning().f4w == 1 : tiles <= (int64_t)cus && nchunks >= 2;
      if (split && lds + 8 * F4_SCALE_SLOT + 512 <= (size_t)F4_LDS_MAX) {
        if (sr_ok) return launch_f4_k<SDT, 8, 0, 1, SR, 1>(a, s, "fp4_tq1_t1_ks", (int)nchunks, lds);
        return launch_f4_k<SDT, 8, 0, 1, 0, 1>(a, s, "fp4_tq1_t1_ks", (int)nchunks, lds);
      }
      const bool four = tuning().f4w ? tuning().f4w == 4 : tiles <= 2 * (int64_t)cus;
      if (four) {
        if (sr_ok && lds + 4 * F4_SCALE_SLOT <= (size_t)F4_LDS_MAX) return launch_f4_k<SDT, 4, 0, 1, SR>(a, s, "fp4_tq1_t1_w4", (int)nchunks, lds);
        return launch_f4_k<SDT, 4>(a, s, "fp4_tq1_t1_w4", (int)nchunks, lds);
      }
    }
    if (sr_ok && lds + 8 * F4_SCALE_SLOT <= (size_t)F4_LDS_MAX) return launch_f4_k<SDT, 8, 0, 1, SR>(a, s, "fp4_tq1_t1_w8", (int)nchunks, lds);
    return launch_f4_k<SDT, 8>(a, s, "fp4_tq1_t1_w8", (int)nchunks, lds);
  }
  if (sr_ok && lds + 16 * F4_SCALE_SLOT <= (size_t)F4_LDS_MAX) return launch_f4_k<SDT, 16, 0, 1, SR>(a, s, "fp4_tq1_t1_w16", (int)nchunks, lds);
  return launch_f4_k<SDT, 16>(a, s, "fp4_tq1_t1_w16", (int)nchunks, lds);
}

}  // namespace

// One token row per expert, or up to 2 / 4 / 6 / 8 (two fp8 pieces per activation), or - when most experts have few
// rows (T <= 4 E) - up to 64 as launches of 8 rows each and the rest: an expert costs what its own rows cost (and
// nothing in a launch whose rows it does not have), so a launch in which a few experts have many rows, or whose
// max_rows is only an upper bound, is not held to that pace.
// BP_ERR_UNSUPPORTED (no message): the caller falls back to its other kernels.
namespace {
template <int SDT>
int launch_f4_rows(const GemmArgs& a, hipStream_t s, int64_t rows, int first_row) {
  if (rows <= 1 && first_row == 0) return launch_f4<SDT, 1>(a, s);
  if (rows <= 2) return launch_f4<SDT, 2>(a, s, first_row);
  if (rows <= 4) return launch_f4<SDT, 4>(a, s, first_row);
  // Seven or eight rows of a large call: four through the streaming kernel and the rest in a second launch of it (measured
  // on 128 x 2048 x 7168: 8 rows 225 against 235 us; 6 rows as four and a pair 206 against 188: they stay below)
  if (SDT != BP_F32 && tuning().tq1 != 'r' && rows >= 7) {
    const int rc = launch_tq1_gemv_cw(a, s, 4, (a.K + 639) / 640, f4_cus(), first_row);
    if (rc == BP_OK) return launch_f4_rows<SDT>(a, s, rows - 4, first_row + 4);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  if (rows <= 6) return launch_f4<SDT, 6>(a, s, first_row);
  return launch_f4<SDT, 8>(a, s, first_row);
}
template <int SDT>
int launch_f4_any(const GemmArgs& a, hipStream_t s) {
  for (int64_t first = 0; first < a.max_rows; first += 8) {
    const int rc = launch_f4_rows<SDT>(a, s, a.max_rows - first < 8 ? a.max_rows - first : 8, (int)first);
    if (rc != BP_OK) return rc;
  }
  return BP_OK;
}
}  // namespace

int launch_tq1_gemv_fp4(const GemmArgs& a, hipStream_t s) {
  if (a.x_dtype != BP_BF16 && a.x_dtype != BP_F16 && a.x_dtype != BP_I8) return BP_ERR_UNSUPPORTED;
  if (a.max_rows > 1 && a.x_dtype == BP_F16) return BP_ERR_UNSUPPORTED;  // (11 significant bits need the third piece)
  int64_t few = 4;  // "most experts have few rows": at most this many routed rows per expert on average
  if (tuning().f4t >= 0) few = tuning().f4t;  // (development)
  if (a.max_rows < 1 || a.max_rows > 64 || (a.max_rows > 8 && a.T > few * a.E)) return BP_ERR_UNSUPPORTED;
  if (a.N % 16 != 0 || a.Kp != (a.K + 4) / 5 || (a.group != 128 && a.group != 256)) return BP_ERR_UNSUPPORTED;
  for (int t = 0; t < a.n_terms; ++t)
    if (a.scale_dtype == BP_F32 && ((uintptr_t)a.w_scale[t] & 3) != 0) return BP_ERR_UNSUPPORTED;
  if (a.max_rows > 8) {  // (both launches must be possible before the first one adds to the output)
    const int64_t nchunks = (a.K + 639) / 640, fit = (F4_LDS_MAX - F4_LUT_BYTES) / (8 * f4_chunk_bytes(8));
    if ((nchunks + fit - 1) / fit > 4) return BP_ERR_UNSUPPORTED;
  }
  if (a.scale_dtype == BP_F16) return launch_f4_any<BP_F16>(a, s);
  if (a.scale_dtype == BP_BF16) return launch_f4_any<BP_BF16>(a, s);
  if (a.scale_dtype == BP_F32) return launch_f4_any<BP_F32>(a, s);
  return BP_ERR_UNSUPPORTED;
}

}  // namespace bp

// TQ2 grouped GEMM for bf16 activations and token tiles of 16 or 32 rows on the scaled fp8 x fp4 matrix instruction
// (v_mfma_scale_f32_16x16x128_f8f6f4), over activations converted beforehand: 2-bit codes become fp4 operands with four
// vector instructions per 16 weights, and one matrix instruction covers exactly one 128-wide scale group.
//
// Contract as everywhere (boilerplate/kernels/ternary_cuda.py:58-63, boilerplate/kernels/csrc/ternary_cuda_kernel.cu:44-99):
// out[t, n] += sum_g scale[n, g] * sum_{k in g} x[t, k] * trit[n, k], float32 accumulation.
//
//  * Weights as fp4. A code u = trit + 1 placed at bits [2:1] of a nibble is the E2M1 number u (0000 = 0, 0010 = 1,
//    0100 = 2), so a packed dword (16 codes) becomes two operand dwords by (w << 1) & 0x66666666 (even codes) and
//    (w >> 1) & 0x66666666 (odd codes): no table, no LDS. The products then carry sum x * u; every group's accumulator
//    starts from -sum x, which leaves sum x * (u - 1). The unused code 3 reads 4 - 1 = +3 (pack never writes it).
//  * A lane loads 16 bytes of its row per 64-byte window (rows are 16-byte aligned: K % 256 == 0); two
//    v_permlane32_swap leave every lane with 8 bytes of each of the window's two groups, so the four lanes of a row
//    supply the 128 weights of ONE group to a matrix instruction: lane quarter kb holds the group's weights
//    64 (kb % 2) + 32 (kb / 2) .. + 31.
//  * Activations as two fp8 (E4M3) pieces under a power-of-two block scale that the instruction applies itself: the
//    32 activations that meet one lane of operand B (32 consecutive k) share one E8M0 scale 2^(e - 7), e the exponent
//    of the block's largest magnitude; y = x / scale = p0 + p1, p0 = y rounded to E4M3, p1 the rounded remainder.
//    bf16 activations are exactly p0 + p1 down to 2^-9 of their block's largest magnitude; less than 2^-17 of it is
//    dropped below. Products fp8 x fp4 are exact. A block that holds a NaN or an infinity makes the token's outputs NaN.
//  * The conversion is vector-ALU work, about as many cycles per token as a workgroup's matrix instructions, and every
//    row block of an expert would repeat it. So it runs once, in a kernel of its own (k_stage_tq2f), into a workspace of
//    the caller: per token tile of 32 and 64-byte window, 17 KiB in exactly the layout the GEMM's LDS buffer has
//    (operands in operand-A register order, block scales, offset sums). The GEMM copies a window's 17 KiB from there.
//  * A GEMM workgroup (8 waves) owns 512 output rows x 32 tokens; a wave 64 rows (4 row tiles) x 32 tokens (2 token
//    tiles): an operand A read from LDS feeds 4 matrix instructions, a decoded weight meets 32 tokens. Weights, scales
//    and staged activations are requested two windows ahead, one load after each row tile's matrix instructions (all at
//    once they fill the CU's vector-memory queue and the waves that come last wait thousands of cycles to issue theirs);
//    every wave issues the same loads in the same order in every window and the stacked terms run as one sequence of
//    windows, so every wait is for loads at least a window old and counts the younger ones exactly. One barrier per window.
//
// TQ1 (FMT = BP_TQ1) runs on the same kernel; only how a lane gets its 32 weights of a group differs. Base-3 bytes have no
// bit fields and groups of 128 digits end inside bytes (128 / 5 = 25.6), so the lane takes the 8 bytes that hold its 32
// digits - bytes floor(t / 5) .. + 7 of its row, t = 128 g + 64 (kb % 2) + 32 (kb / 2) the slice's first digit - looks each
// up in a table byte -> 5 fp4 codes (-1, 0, +1 as E2M1; 20 bits; one copy per lane in LDS, so the address is one
// v_perm_b32 and no two lanes share a bank), strings the 8 entries together to 160 bits and shifts them right by the
// 0..4 digits the slice starts inside its first byte (4 v_alignbit_b32): 128 bits = the lane's operand B in k order, one
// matrix instruction per scale group. The codes are signed: no offset sums. The staged activations are the same, with
// the 16 activations of a thread in consecutive bytes instead of TQ2's even / odd order.
// A window's bytes come from memory the way the cache likes them, not the way the matrix instruction wants them: four
// neighbouring lanes load the 64 bytes (at a dword-aligned address) that hold a row's 51.2 bytes of the window - 16
// cache requests per wave load, where a load in the instruction's own lane order (neighbouring lanes = different rows)
// makes 64 and one of 8 unaligned bytes per lane more still; the L1's tag rate of about one request per clock was what
// the kernel ran at. The 16 x 64 bytes go through a per-wave transit area in LDS (row pitch 72), from which a lane reads
// the three dwords around its slice and shifts them into place (2 v_alignbyte_b32).
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
using FC = std::integral_constant<int, V>;

constexpr int F_WAVES = 8;                         // waves per workgroup
constexpr int F_RT = 4;                            // 16-row tiles per wave
constexpr int F_THREADS = F_WAVES * 64;
constexpr int F_ROWS = F_WAVES * 16 * F_RT;        // output rows per workgroup
constexpr int F_OPS = 2 * 2 * 2 * 2048;            // operands of a window: 2 groups x 2 token tiles x 2 pieces x 2 KiB
constexpr int F_SCL = 2 * 64 * 4;                  // ... the block scales: per token tile one dword per lane (byte g = group g)
constexpr int F_SUM = 2 * 32 * 4;                  // ... and the offset sums: [group][token] float
constexpr int F_TAIL = F_SCL + F_SUM;              // (48 x 16 bytes)
constexpr int F_FB = 32 * 544;                     // a staged window of a token tile: operands, scales, sums, padding (544 bytes per token: a multiple of 16)
static_assert(F_OPS + F_TAIL <= F_FB && F_OPS == F_THREADS * 32 && F_TAIL % 16 == 0, "a staged window: two 16-byte pieces per thread and a tail");
constexpr int F_SC = 2 * F_FB;                     // LDS: two staged windows, then the rows' scales: 2 slots of [512 rows][8 scales] as stored
constexpr int f_lds_bytes(int scale_bytes) { return F_SC + 2 * F_ROWS * 8 * scale_bytes; }  // 51,200 (16-bit scales) / 67,584 (float32)
constexpr int F_LUT = 256 * 256;                   // TQ1: the byte table at LDS address 0 (entry v, copy c at 256 v + 4 c), everything else behind it
constexpr int F_TP = 72;                           // TQ1: pitch of a row's 64 bytes in the transit area (18 dwords: 16 rows start in 16 different banks), and the area of a wave's row tile
constexpr int F_TR = 16 * F_TP;

template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(FC<N - 1>{});
  }
}

// Where token tile (expert e, first row tok0) keeps its staged windows: tile z of expert e starts 32 (e + z) + offsets[e]
// tokens into the workspace, so tiles never overlap whatever the experts' row counts are.
__device__ __forceinline__ unsigned char* staged_tile(const GemmArgs& a, int64_t e, int64_t tok0) {
  return a.stage + (tok0 + 32 * e) * (a.K / 256) * (F_FB / 32);
}

// ---- the conversion: one workgroup per (token tile, window). Wave = (token tile stt, group sg of the window, token half
// mh); lane = (token m3 of 8, quarter kbA of operand A's lanes, half hi of its registers): the thread converts the 16
// activations that fill registers 4 hi .. 4 hi + 3 of A lane (m, kbA) for the group's instruction: k = 64 (kbA / 2) +
// 32 hi + 16 (kbA % 2) .. + 15 of the group. A token's group is the 8 lanes (kbA, hi) of one wave: 256 consecutive bytes.
// NAT: activation j of the thread's 16 goes to register j / 4, byte j % 4 (operand B in k order: TQ1); otherwise to
// register 2 (j % 2) + j / 8, byte (j % 8) / 2 (operand B as the even and the odd codes of a packed TQ2 dword).
template <bool NAT>
__global__ __launch_bounds__(F_THREADS) void k_stage_tq2f(GemmArgs a) {
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const TileRef tr = tile_ref(a, blockIdx.x, blockIdx.z);
  if (!tr.live) return;  // uniform for the workgroup
  const int64_t tok0 = tr.tok0;
  const int ntok = (int)(tr.o1 - tok0 < 32 ? tr.o1 - tok0 : 32);
  const int s = blockIdx.y;  // the window
  const int stt = wave & 1, sg = (wave >> 1) & 1, mh = wave >> 2;
  const int m3 = lane & 7, kbA = (lane >> 3) & 3, hi = lane >> 5;
  const int sm = 8 * mh + m3;
  unsigned char* dst = staged_tile(a, tr.e, tok0) + (int64_t)s * F_FB;
  if (stt == 1 && ntok <= 16) {  // no second token tile: its scales and sums are read all the same (and multiply nothing that is stored)
    if ((kbA & 1) == 0) dst[F_OPS + (stt * 64 + ((kbA >> 1) + 2 * hi) * 16 + sm) * 4 + sg] = 127;
    if (kbA == 0 && hi == 0) *(float*)(dst + F_OPS + F_SCL + (sg * 32 + 16 * stt + sm) * 4) = 0.f;
    return;
  }
  int srow = 16 * stt + sm;
  if (srow >= ntok) srow = ntok - 1;  // rows past the expert's tokens repeat its last one (their results are not stored)
  int64_t xrow = tok0 + srow;
  if (a.x_index) xrow = clamp_i64(a.x_index[xrow] / a.x_div, 0, a.x_rows - 1);  // (the routed row's token)
  const uint16_t* xp = (const uint16_t*)a.x + xrow * a.K + 256 * (int64_t)s + 128 * sg + 64 * (kbA >> 1) + 32 * hi + 16 * (kbA & 1);
  const u32x4 raw[2] = {*(const u32x4*)xp, *(const u32x4*)(xp + 8)};
  float y[16];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const unsigned v = raw[i >> 2][i & 3];
    y[2 * i] = __uint_as_float(v << 16);
    y[2 * i + 1] = __uint_as_float(v & 0xffff0000u);
  }
  unsigned mx = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const unsigned v = __float_as_uint(y[i]) & 0x7fffffffu;
    mx = mx > v ? mx : v;
  }
  {  // the block of 32 = this lane's 16 and those of the lane with the other kbA % 2
    const unsigned other = (unsigned)__shfl_xor((int)mx, 8, 64);
    mx = mx > other ? mx : other;
  }
  const int ex = (int)(mx >> 23);
  int sh = 134 - ex;  // brings the block's largest magnitude into [128, 256)
  sh = sh > 126 ? 126 : sh;
  float mult = __uint_as_float((unsigned)(127 + sh) << 23);
  if (ex == 255) mult = __uint_as_float(0x7fc00000u);  // a NaN or an infinity in the block: every slot becomes NaN
  u32x4 p0, p1;
  float used = 0.f;  // sum of what the two pieces represent, in the block's scaled domain
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int v1 = d >> 1, v0 = d & 1;
    int c0 = 0, c1 = 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float f0 = y[NAT ? 4 * d + 2 * h : 8 * v0 + 4 * h + v1] * mult, f1 = y[NAT ? 4 * d + 2 * h + 1 : 8 * v0 + 4 * h + 2 + v1] * mult;
      c0 = h == 0 ? __builtin_amdgcn_cvt_pk_fp8_f32(f0, f1, c0, false) : __builtin_amdgcn_cvt_pk_fp8_f32(f0, f1, c0, true);
      const float b0 = h == 0 ? __builtin_amdgcn_cvt_f32_fp8(c0, 0) : __builtin_amdgcn_cvt_f32_fp8(c0, 2);
      const float b1 = h == 0 ? __builtin_amdgcn_cvt_f32_fp8(c0, 1) : __builtin_amdgcn_cvt_f32_fp8(c0, 3);
      const float r0 = f0 - b0, r1 = f1 - b1;
      c1 = h == 0 ? __builtin_amdgcn_cvt_pk_fp8_f32(r0, r1, c1, false) : __builtin_amdgcn_cvt_pk_fp8_f32(r0, r1, c1, true);
      const float e0 = h == 0 ? __builtin_amdgcn_cvt_f32_fp8(c1, 0) : __builtin_amdgcn_cvt_f32_fp8(c1, 2);
      const float e1 = h == 0 ? __builtin_amdgcn_cvt_f32_fp8(c1, 1) : __builtin_amdgcn_cvt_f32_fp8(c1, 3);
      used += (b0 + e0) + (b1 + e1);
    }
    p0[d] = (unsigned)c0;
    p1[d] = (unsigned)c1;
  }
  unsigned char* ob = dst + ((sg * 2 + stt) * 2) * 2048 + (kbA * 2 + hi) * 256 + sm * 16;
  *(u32x4*)ob = p0;
  *(u32x4*)(ob + 2048) = p1;
  // the block's scale: byte sg of the scale operand's dword in lane (m, kb) with kb % 2 = kbA / 2, kb / 2 = hi
  if ((kbA & 1) == 0) dst[F_OPS + (stt * 64 + ((kbA >> 1) + 2 * hi) * 16 + sm) * 4 + sg] = (unsigned char)(127 - sh);
  // the group's offset sum: what the pieces represent, back in the activations' units, over the token's 8 lanes
  float part = used * __uint_as_float((unsigned)(127 - sh) << 23);
  if (ex == 255) part = __uint_as_float(0x7fc00000u);
  part += __shfl_xor(part, 8, 64);
  part += __shfl_xor(part, 16, 64);
  part += __shfl_xor(part, 32, 64);
  if (kbA == 0 && hi == 0) *(float*)(dst + F_OPS + F_SCL + (sg * 32 + 16 * stt + sm) * 4) = -part;
}

// GS = 1: scale groups of 256 (the two groups of a window share a scale); 0: of 128.
template <int SDT, int FMT, int GS>
__global__ __launch_bounds__(F_THREADS, 2) void k_gemm_tq2f(GemmArgs a) {
  constexpr int SB = SDT == BP_F32 ? 4 : 2;
  constexpr bool Q1 = FMT == BP_TQ1;
  constexpr unsigned LB = Q1 ? F_LUT : 0;  // LDS address of the staged windows

  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;
  const int r16 = lane & 15, kb = lane >> 4;
  // SwiGLU in the epilogue: the launch's rows are NH gate rows followed by NH up rows, and a wave's four row tiles are two
  // of the gate (r = 0, 1) and the same two of the up projection (r = 2, 3): a row block covers F_ROWS / 2 of either
  const bool glu = a.glu_h != nullptr;
  const int64_t NH = glu ? a.N / 2 : a.N;
  const int row_blocks = glu ? (int)((NH + F_ROWS / 2 - 1) / (F_ROWS / 2)) : (int)((a.N + F_ROWS - 1) / F_ROWS);
  int wg_block;
  const TileRef tr = tile_of_workgroup(a, blockIdx.x, row_blocks, wg_block);
  if (!tr.live) return;  // uniform for the workgroup
  const int64_t e = tr.e, tok0 = tr.tok0, o1 = tr.o1;
  const int ntok = (int)(o1 - tok0 < 32 ? o1 - tok0 : 32);
  const bool two = ntok > 16;  // the second token tile holds tokens
  // first row of row tile r of wave wv (-1: past the rows)
  auto tile_row = [&](int wv, int r) -> int64_t {
    if (glu) {
      const int64_t c = (int64_t)wg_block * (F_ROWS / 2) + wv * (8 * F_RT) + 16 * (r & 1);
      return c < NH ? (r >> 1) * NH + c : -1;
    }
    const int64_t row = (int64_t)wg_block * F_ROWS + wv * (16 * F_RT) + 16 * r;
    return row < a.N ? row : -1;
  };

  const int nwin = (int)(a.K / 256);      // 64-byte windows of a row = pairs of 128-wide groups
  const int NW = nwin * a.n_terms;        // the stacked terms, one after the other
  constexpr int gs = GS;

  const unsigned alane = LB + (unsigned)(kb * 512 + r16 * 16);
  if constexpr (Q1) {  // the byte table: two threads per byte value, 32 copies each
    unsigned v = threadIdx.x >> 1, ent = 0;
    if (v < 243) {
#pragma unroll
      for (int d = 0; d < 5; ++d) {
        const unsigned q = v / 3, dig = v - 3 * q;
        ent |= (dig == 0 ? 0xAu : dig == 2 ? 0x2u : 0u) << (4 * d);
        v = q;
      }
    }
#pragma unroll
    for (int c = 0; c < 32; ++c) *(lds_u32*)(256u * (threadIdx.x >> 1) + 128u * (threadIdx.x & 1) + 4u * c) = ent;
  }
  const unsigned lane4 = (unsigned)lane << 2;
  int ones = 0x7f7f7f7f;  // operand B's block scales: 2^0
  asm volatile("" : "+v"(ones));
  unsigned m66 = 0x66666666u;
  asm volatile("" : "+s"(m66));

  // ---- the load stream. Window w of the sequence is window w % nwin of term w / nwin; (lterm, ls) names the next window
  // to request. Per window every wave issues, in this order: the thread's three pieces of the staged window, the thread's
  // row's two scales, the wave's four weight loads. Requests past the last window repeat it (never used).
  const unsigned voff = (unsigned)r16 * (unsigned)a.Kp + 16u * kb;
  // TQ1: first digit of the lane's slice of a window's first group (the second group's: + 128)
  const unsigned cg0 = 64u * (kb & 1) + 32u * (kb >> 1);
  auto slice_of = [&](unsigned s, unsigned g, unsigned& first_byte, unsigned& digit) {  // of window s of a term: byte offset past floor(256 s / 5), digit 0..4 inside it
    const unsigned rho = 256u * s - 5u * ((256u * s) / 5u);
    const unsigned x = rho + cg0 + 128u * g;  // < 1024: x / 5 = x * 205 >> 10
    first_byte = (x * 205u) >> 10;
    digit = x - 5u * first_byte;
  };
  unsigned wrow[F_RT];  // byte offset of the row tile's first row (a tile past N repeats the wave's first tile and is not stored)
#pragma unroll
  for (int r = 0; r < F_RT; ++r) {
    int64_t row = tile_row(wave, r);
    if (row < 0) row = tile_row(wave, 0) < 0 ? 0 : tile_row(wave, 0);
    wrow[r] = (unsigned)(row * a.Kp);
  }
  // TQ1: the expert's rows as a buffer with a dword-aligned base (mis = what the rows' first byte is past it; the same
  // for every term: a precondition). Loading lane L takes piece L % 4 of row L / 4 of a tile: lpre[r] = byte offset of
  // that piece for window 0, before alignment. Reading lane (r16, kb): upre[r] = byte offset of its row (the low two
  // bits of it and the window's first byte say where the row's bytes start in its 64-byte image).
  const unsigned mis = Q1 ? (unsigned)((uintptr_t)(a.packed[0] + e * a.N * a.Kp) & 3) : 0u;
  unsigned lpre[F_RT], upre[F_RT];
#pragma unroll
  for (int r = 0; r < F_RT; ++r) {
    lpre[r] = mis + wrow[r] + (unsigned)(lane >> 2) * (unsigned)a.Kp + 16u * (lane & 3);
    upre[r] = mis + wrow[r] + (unsigned)r16 * (unsigned)a.Kp;
  }
  unsigned lq = 0;  // first byte of the window to request: floor(256 ls / 5)
  const unsigned TRW = LB + (unsigned)f_lds_bytes(SB) + (unsigned)(wave * F_RT * F_TR);  // the wave's transit area
  const int64_t my_tile = tile_row((int)(threadIdx.x >> 6), (int)((threadIdx.x >> 4) & 3));  // thread = row, in the order the waves hold their row tiles
  const unsigned my_scales = my_tile >= 0 ? (unsigned)((my_tile + (threadIdx.x & 15)) * a.G * SB) : 0xfffffff0u;  // rows past N: zeros
  const __amdgpu_buffer_rsrc_t xrs = make_rsrc(staged_tile(a, e, tok0), (int64_t)nwin * F_FB);
  const unsigned tail_off = threadIdx.x < F_TAIL / 16 ? (unsigned)(F_OPS + 16 * threadIdx.x) : 0xfffffff0u;  // (past the range: no memory access)
  int lterm = 0, ls = 0;
  __amdgpu_buffer_rsrc_t wrs, srs;
  auto set_term = [&](int term) {
    const unsigned char* wbeg = a.packed[term];
    // (TQ1: the range ends with the dword that holds the tensor's last byte - a dword that straddled the end of the range
    // would read as zero, valid bytes included; up to 3 bytes behind the tensor are read with it, inside a dword of which
    // the tensor owns a byte, and never used; whole dwords past that read as zero)
    wrs = make_rsrc(wbeg + e * a.N * a.Kp - mis, Q1 ? (((a.E - e) * a.N * a.Kp + mis + 3) & ~(int64_t)3) : (a.E - e) * a.N * a.Kp);
    const unsigned char* sbeg = (const unsigned char*)a.w_scale[term];
    const unsigned char* expert_scales = sbeg + e * a.N * a.G * SB;
    srs = make_rsrc(expert_scales, (sbeg + a.E * a.N * a.G * SB) - expert_scales);
  };
  set_term(0);
  u32x4 W[2][F_RT];        // the weights of the windows of either parity
  u32x4 xa[2][3];          // ... the thread's pieces of their staged activations (two of the operands, one of the tail)
  // The rows' scales travel in blocks of 8 entries (4 windows, or 8 with one scale per 256 weights): thread = row, one
  // 16- or 32-byte load per block (a load per window of 4 bytes per lane costs the memory pipeline as much as one of 16,
  // and fetches a 64-byte sector per row each time). A row's last block starts 8 entries before the row's end.
  u32x4 sq[SB / 2];        // the thread's row's block on its way to LDS
  auto scale_block = [&](int sw, unsigned& first) {  // the block of window sw of a term and its first entry
    const unsigned b = (unsigned)((2 * sw) >> gs) >> 3;
    first = 8u * b + 8u <= (unsigned)a.G ? 8u * b : (unsigned)a.G - 8u;
    return b;
  };
  auto starts_block = [&](int sw) { return ((((unsigned)(2 * sw)) >> gs) & 7u) == 0u; };
  // part 0..3: the weights of row tile `part`; 4: the scales; 5, 6, 7: the staged activations; 8: on to the next window.
  // Order within a window: 5, 6, 7, 4 (with the first group's matrix instructions), 0 .. 3 (with the second group's), 8.
  auto request = [&](auto p_c, auto part_c) {
    constexpr int P = decltype(p_c)::value, PART = decltype(part_c)::value;
    const unsigned s = (unsigned)ls;
    if constexpr (PART < F_RT && !Q1) W[P][PART] = buf_load16(wrs, voff, wrow[PART] + 64u * s);
    if constexpr (PART < F_RT && Q1) W[P][PART] = buf_load16(wrs, (lpre[PART] + lq) & ~3u, 0u);
    if (PART == 4) {
      if (starts_block((int)s)) {  // uniform
        unsigned first;
        scale_block((int)s, first);
        const unsigned so = my_scales == 0xfffffff0u ? my_scales : my_scales + first * SB;
#pragma unroll
        for (int i = 0; i < SB / 2; ++i) sq[i] = buf_load16(srs, so == 0xfffffff0u ? so : so + 16u * i, 0u);
      }
    }
    if constexpr (PART == 5 || PART == 6) xa[P][PART - 5] = buf_load16(xrs, 16u * threadIdx.x + 8192u * (PART - 5), (unsigned)F_FB * s);
    if (PART == 7) xa[P][2] = buf_load16(xrs, tail_off, (unsigned)F_FB * s);
    if (PART == 8) {
      if (ls + 1 < nwin) ++ls;
      else if (lterm + 1 < a.n_terms) {
        ++lterm;
        ls = 0;
        set_term(lterm);
      }
      if constexpr (Q1) lq = (256u * (unsigned)ls) / 5u;
    }
  };
  auto request_all = [&](auto p_c) {
    request(p_c, FC<5>{});
    request(p_c, FC<6>{});
    request(p_c, FC<7>{});
    request(p_c, FC<4>{});
    static_for<F_RT>([&](auto r_c) { request(p_c, r_c); });
    request(p_c, FC<8>{});
  };
  auto staged_store = [&](int buf, const u32x4 (&v)[3]) {
    const unsigned ab = LB + (unsigned)(buf * F_FB);
    *(lds_u32x4*)(ab + 16u * threadIdx.x) = v[0];
    *(lds_u32x4*)(ab + 8192u + 16u * threadIdx.x) = v[1];
    if (threadIdx.x < F_TAIL / 16) *(lds_u32x4*)(ab + (unsigned)F_OPS + 16u * threadIdx.x) = v[2];
  };
  // The two LDS slots alternate block by block (also from a term's last block to the next term's first): the slot
  // written before a window's barrier was last read two blocks - at least four barriers - earlier.
  int wslot = 0, rslot = 0, rslot_next = 0;  // (uniform)
  auto scale_store = [&](int sw) {  // the block that window sw of a term starts, if it starts one
    if (!starts_block(sw)) return;  // uniform
#pragma unroll
    for (int i = 0; i < SB / 2; ++i) *(lds_u32x4*)(LB + (unsigned)(F_SC + (wslot * F_ROWS + (int)threadIdx.x) * (8 * SB) + 16 * i)) = sq[i];
    rslot_next = wslot;
    wslot ^= 1;
  };

  auto all_windows = [&](auto tt_c) {
    constexpr int TT = decltype(tt_c)::value;  // token tiles processed
    f32x4 total[F_RT][TT];
#pragma unroll
    for (int r = 0; r < F_RT; ++r)
#pragma unroll
      for (int t = 0; t < TT; ++t) total[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- prologue: windows 0 and 1 requested, window 0's operands and scales into LDS
    request_all(FC<0>{});
    request_all(FC<1>{});
    staged_store(0, xa[0]);
    scale_store(0);
    __syncthreads();

    // ---- The matrix instructions of a wave run on without a gap. A group's go in batches of four row tiles - (token
    // tile 0, piece 0), (1, 0), (0, 1), (1, 1); with one token tile only the first and the third - so that an operand A
    // is free for the next group's (read from LDS behind its batch) as soon as its batch has issued, an instruction of
    // the second pieces finds its accumulator finished, and the scaling of token tile 0's sums runs beside batch 3, that
    // of the last token tile's beside the next group's batch 0. The workgroup's one barrier per window sits between the two groups: before
    // it a wave writes the next window's staged activations and scales to LDS, after it it reads them.
    constexpr int DT = TT - 1;       // the token tile whose sums wait for the next group's batch 0
    i32x8 A[TT][2];
    f32x4 base[TT];
    int sa[2][TT];                   // [window parity][token tile]
    unsigned sraw[2][F_RT][SB / 2];  // [window parity]: the window's two scales of the lane's row of each row tile, as stored
    float scp[F_RT];                 // the scales of the group whose token tile DT is still to be summed
    f32x4 C[F_RT][TT];
    i32x8 B[F_RT];
#pragma unroll
    for (int r = 0; r < F_RT; ++r) {
      scp[r] = 0.f;
#pragma unroll
      for (int t = 0; t < TT; ++t) C[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    auto read_a = [&](unsigned ab, int g, auto t_c, auto p_c) {
      constexpr int t = decltype(t_c)::value, pp = decltype(p_c)::value;
      const unsigned at = ab + (unsigned)(((g * 2 + t) * 2 + pp) * 2048) + alane;
      const u32x4 lo = *(const lds_u32x4*)at, hi4 = *(const lds_u32x4*)(at + 256);
      A[t][pp] = i32x8{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi4.x, (int)hi4.y, (int)hi4.z, (int)hi4.w};
    };
    auto read_base = [&](unsigned ab, int g) {
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        if constexpr (Q1) base[t] = f32x4{0.f, 0.f, 0.f, 0.f};  // (signed codes: nothing to take off)
        else base[t] = __builtin_bit_cast(f32x4, *(const lds_u32x4*)(ab + F_OPS + F_SCL + (unsigned)((g * 32 + 16 * t + 4 * kb) * 4)));
      }
    };
    auto read_window_scales = [&](auto h_c, int sw) {  // block scales and row scales of the window of parity H, window sw of its term
      constexpr int H = decltype(h_c)::value;
      const unsigned ab = LB + (unsigned)(H * F_FB);
      unsigned first;
      scale_block(sw, first);
      if (starts_block(sw)) rslot = rslot_next;
      const unsigned sb = LB + (unsigned)(F_SC + (rslot * F_ROWS + wave * (16 * F_RT) + r16) * (8 * SB)) + ((((unsigned)(2 * sw)) >> gs) - first) * SB;
#pragma unroll
      for (int t = 0; t < TT; ++t) sa[H][t] = (int)*(const lds_u32*)(ab + F_OPS + (unsigned)((t * 64 + lane) * 4));
#pragma unroll
      for (int r = 0; r < F_RT; ++r) {
        const unsigned at = sb + (unsigned)(16 * r * 8 * SB);
        if (SB == 2) {
          if (gs) sraw[H][r][0] = (unsigned)*(const lds_u16*)at * 0x10001u;  // (one scale for both groups)
          else sraw[H][r][0] = *(const lds_u32*)at;
        } else if (gs) {
          sraw[H][r][0] = sraw[H][r][SB / 2 - 1] = *(const lds_u32*)at;
        } else {
          const u32x2 v = *(const lds_u32x2*)at;
          sraw[H][r][0] = v.x;
          sraw[H][r][SB / 2 - 1] = v.y;
        }
      }
    };
    read_a(0u, 0, FC<0>{}, FC<0>{});
    read_a(0u, 0, FC<0>{}, FC<1>{});
    if constexpr (TT == 2) {
      read_a(0u, 0, FC<1>{}, FC<0>{});
      read_a(0u, 0, FC<1>{}, FC<1>{});
    }
    read_base(0u, 0);
    read_window_scales(FC<0>{}, 0);

    unsigned D[F_RT][2][2];  // TQ2: the window's bytes regrouped: D[r][g] = the lane's 8 bytes (32 weights) of group g
    // TQ1: operand B of a group is made while the group before it is multiplied, in three steps per row tile, each
    // behind the matrix instructions of another batch so that no wave waits for the LDS between a read and its use:
    // the three dwords around the lane's slice are read from the transit area (T), shifted into place and looked up in
    // the table (L), and the 8 entries strung together (S). Bq[g % 2]: the operands of group g; tb, en: dwords and table
    // entries on their way; shq[0 / 1] / fbq[0 / 1]: of this window's group 0 / 1, the bits by which the 160-bit string
    // is shifted (4 x the digit the lane's slice starts at inside its first byte) and the slice's first byte past the
    // window's; [2]: of the next window's group 0. ucur / unxt[r]: where the lane's row starts in its 64-byte image
    // (0..3) in this window / the next.
    u32x4 Bq[2][F_RT];
    unsigned en[2][8], tb[2][3];
    unsigned shq[3] = {0u, 0u, 0u}, fbq[3] = {0u, 0u, 0u}, ucur[F_RT], unxt[F_RT];
    auto transit_write = [&](const u32x4 (&w4)[F_RT]) {  // a window's 4 x 16 x 64 bytes, row by row
#pragma unroll
      for (int r = 0; r < F_RT; ++r) {  // (the pitch is a multiple of 8, not of 16: two 8-byte stores)
        const unsigned at = TRW + (unsigned)(r * F_TR) + (unsigned)((lane >> 2) * F_TP + 16 * (lane & 3));
        *(lds_u32x2*)at = u32x2{w4[r].x, w4[r].y};
        *(lds_u32x2*)(at + 8u) = u32x2{w4[r].z, w4[r].w};
      }
    };
    auto transit_read = [&](unsigned (&t3)[3], int r, unsigned off) {  // the dwords that hold bytes off .. off + 7 of the lane's row of tile r
      const unsigned at = TRW + (unsigned)(r * F_TR) + (unsigned)(r16 * F_TP) + (off & ~3u);
      t3[0] = *(const lds_u32*)at;
      t3[1] = *(const lds_u32*)(at + 4u);
      t3[2] = *(const lds_u32*)(at + 8u);
    };
    auto lookups = [&](unsigned (&e8)[8], const unsigned (&t3)[3], unsigned off) {  // byte i of the slice -> its 5 codes: address = 256 byte + 4 lane
      const unsigned d0 = __builtin_amdgcn_alignbyte(t3[1], t3[0], off), d1 = __builtin_amdgcn_alignbyte(t3[2], t3[1], off);
      e8[0] = *(const lds_u32*)__builtin_amdgcn_perm(d0, lane4, 0x0c0c0400u);
      e8[1] = *(const lds_u32*)__builtin_amdgcn_perm(d0, lane4, 0x0c0c0500u);
      e8[2] = *(const lds_u32*)__builtin_amdgcn_perm(d0, lane4, 0x0c0c0600u);
      e8[3] = *(const lds_u32*)__builtin_amdgcn_perm(d0, lane4, 0x0c0c0700u);
      e8[4] = *(const lds_u32*)__builtin_amdgcn_perm(d1, lane4, 0x0c0c0400u);
      e8[5] = *(const lds_u32*)__builtin_amdgcn_perm(d1, lane4, 0x0c0c0500u);
      e8[6] = *(const lds_u32*)__builtin_amdgcn_perm(d1, lane4, 0x0c0c0600u);
      e8[7] = *(const lds_u32*)__builtin_amdgcn_perm(d1, lane4, 0x0c0c0700u);
    };
    auto strung = [&](const unsigned (&e8)[8], unsigned sh) {  // 8 x 20 bits in a row, shifted right by sh < 32 bits: the low 128
      const unsigned c0 = e8[0] | (e8[1] << 20);
      const unsigned c1 = (e8[1] >> 12) | (e8[2] << 8) | (e8[3] << 28);
      const unsigned c2 = (e8[3] >> 4) | (e8[4] << 16);
      const unsigned c3 = (e8[4] >> 16) | (e8[5] << 4) | (e8[6] << 24);
      const unsigned c4 = (e8[6] >> 8) | (e8[7] << 12);
      return u32x4{__builtin_amdgcn_alignbit(c1, c0, sh), __builtin_amdgcn_alignbit(c2, c1, sh),
                   __builtin_amdgcn_alignbit(c3, c2, sh), __builtin_amdgcn_alignbit(c4, c3, sh)};
    };
    auto window_slices = [&](int sw, int sn) {  // of window sw of a term, and of group 0 of the window after it
#pragma unroll
      for (unsigned g = 0; g < 3; ++g) {
        unsigned dg;
        slice_of((unsigned)(g == 2 ? sn : sw), g & 1, fbq[g], dg);
        shq[g] = 4u * dg;
      }
      const unsigned qc = (256u * (unsigned)sw) / 5u, qn = (256u * (unsigned)sn) / 5u;
#pragma unroll
      for (int r = 0; r < F_RT; ++r) {
        ucur[r] = (upre[r] + qc) & 3u;
        unxt[r] = (upre[r] + qn) & 3u;
      }
    };
    if constexpr (Q1) {  // the first group's operands (window 0 of term 0 has arrived with the prologue's barrier)
      window_slices(0, 0);
      transit_write(W[0]);
#pragma unroll
      for (int r = 0; r < F_RT; ++r) {
        transit_read(tb[r & 1], r, ucur[r] + fbq[0]);
        lookups(en[r & 1], tb[r & 1], ucur[r] + fbq[0]);
        Bq[0][r] = strung(en[r & 1], shq[0]);
      }
    }
    int cs = 0, ns = 0;  // the window's index in its term, and the next window's (uniform)
    auto pgroup = [&](auto h_c, auto g_c) {
      constexpr int H = decltype(h_c)::value, g = decltype(g_c)::value;
      const unsigned nb = (unsigned)((g == 0 ? H : H ^ 1) * F_FB);  // where the next group's operands are (relative to the first staged window)
      constexpr int ng = g ^ 1;
      auto mfma = [&](const i32x8& av, const i32x8& bv, const f32x4& cv, int sav) {
        return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(av, bv, cv, 0 /* A: E4M3 */, 4 /* B: E2M1 */, g, sav, 0, ones);
      };
      auto row_scale = [&](int r) {
        if (SDT == BP_F32) return __uint_as_float(sraw[H][r][g == 0 ? 0 : SB / 2 - 1]);
        const unsigned rawsc = g == 0 ? sraw[H][r][0] & 0xffffu : sraw[H][r][0] >> 16;
        return SDT == BP_F16 ? f16_bits_to_f32((uint16_t)rawsc) : __uint_as_float(rawsc << 16);
      };
      // batch 0: (token tile 0, piece 0). A row tile's operand B is made just before its first use; the previous
      // group's token tile 1 is summed here.
      // TQ1: the next group's operands on their way: group 1 of this window, or group 0 of the next one, whose bytes go
      // into the transit area first (the area's previous content, this window's, was last read in the group before)
      const unsigned sh_next = shq[g == 0 ? 1 : 2], fb_next = fbq[g == 0 ? 1 : 2];
      auto step_t = [&](int slot, int r) { transit_read(tb[slot], r, (g == 0 ? ucur[r] : unxt[r]) + fb_next); };
      auto step_l = [&](int slot, int r) { lookups(en[slot], tb[slot], (g == 0 ? ucur[r] : unxt[r]) + fb_next); };
      if constexpr (Q1 && g == 1) transit_write(W[H ^ 1]);
      static_for<F_RT>([&](auto r_c) {
        constexpr int r = decltype(r_c)::value;
        if constexpr (Q1) {
          B[r] = i32x8{(int)Bq[g][r].x, (int)Bq[g][r].y, (int)Bq[g][r].z, (int)Bq[g][r].w, 0, 0, 0, 0};
        } else {
          const unsigned d0 = D[r][g][0], d1 = D[r][g][1];
          B[r] = i32x8{(int)((d0 << 1) & m66), (int)((d0 >> 1) & m66), (int)((d1 << 1) & m66), (int)((d1 >> 1) & m66), 0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) total[r][DT][i] += scp[r] * C[r][DT][i];
        asm volatile("" : "+v"(total[r][DT]));
        C[r][0] = mfma(A[0][0], B[r], base[0], sa[H][0]);
        asm volatile("" : "+v"(C[r][0]) : : "memory");
        if constexpr (Q1 && r >= 2) step_t(r - 2, r - 2);
        __builtin_amdgcn_sched_barrier(0);
      });
      read_a(nb, ng, FC<0>{}, FC<0>{});
      if (g == 0) staged_store(H ^ 1, xa[H ^ 1]);  // (the other buffer: last read before the previous barrier)
      request(h_c, FC<g == 0 ? 5 : 0>{});
      __builtin_amdgcn_sched_barrier(0);
      // batch 1: (1, 0)
      if constexpr (TT == 2) {
        static_for<F_RT>([&](auto r_c) {
          constexpr int r = decltype(r_c)::value;
          C[r][1] = mfma(A[1][0], B[r], base[1], sa[H][1]);
          asm volatile("" : "+v"(C[r][1]) : : "memory");
          if constexpr (Q1 && r < 2) step_l(r, r);
          if constexpr (Q1 && r >= 2) step_t(r - 2, r);
          __builtin_amdgcn_sched_barrier(0);
        });
        read_a(nb, ng, FC<1>{}, FC<0>{});
      } else if constexpr (Q1) {
        step_l(0, 0);
        step_l(1, 1);
        step_t(0, 2);
        step_t(1, 3);
      }
      if (g == 0) scale_store(ns);
      request(h_c, FC<g == 0 ? 6 : 1>{});
      __builtin_amdgcn_sched_barrier(0);
      // batch 2: (0, 1)
      static_for<F_RT>([&](auto r_c) {
        constexpr int r = decltype(r_c)::value;
        C[r][0] = mfma(A[0][1], B[r], C[r][0], sa[H][0]);
        asm volatile("" : "+v"(C[r][0]) : : "memory");
        if constexpr (Q1 && r < 2) Bq[ng][r] = strung(en[r], sh_next);
        if constexpr (Q1 && r >= 2) step_l(r - 2, r);
        __builtin_amdgcn_sched_barrier(0);
      });
      read_a(nb, ng, FC<0>{}, FC<1>{});
      read_base(nb, ng);  // (the accumulators' starting values were last read by batch 1)
      if (g == 1) read_window_scales(FC<H ^ 1>{}, ns);
      request(h_c, FC<g == 0 ? 7 : 2>{});
      __builtin_amdgcn_sched_barrier(0);
      // batch 3: (1, 1), and token tile 0's sums under the rows' scales
      if constexpr (TT == 2) {
        static_for<F_RT>([&](auto r_c) {
          constexpr int r = decltype(r_c)::value;
          C[r][1] = mfma(A[1][1], B[r], C[r][1], sa[H][1]);
          asm volatile("" : "+v"(C[r][1]) : : "memory");
          const float sc = row_scale(r);
#pragma unroll
          for (int i = 0; i < 4; ++i) total[r][0][i] += sc * C[r][0][i];
          asm volatile("" : "+v"(total[r][0]));
          scp[r] = sc;
          if constexpr (Q1 && r >= 2) Bq[ng][r] = strung(en[r - 2], sh_next);
          __builtin_amdgcn_sched_barrier(0);
        });
        read_a(nb, ng, FC<1>{}, FC<1>{});
      } else {
#pragma unroll
        for (int r = 0; r < F_RT; ++r) scp[r] = row_scale(r);
        if constexpr (Q1) {
          Bq[ng][2] = strung(en[0], sh_next);
          Bq[ng][3] = strung(en[1], sh_next);
        }
      }
      request(h_c, FC<g == 0 ? 4 : 3>{});
      if (g == 1) request(h_c, FC<8>{});
      __builtin_amdgcn_sched_barrier(0);
    };
    auto pwindow = [&](auto h_c) {
      constexpr int H = decltype(h_c)::value;
#pragma unroll
      for (int r = 0; r < F_RT; ++r) {  // (in place: the registers of W[H] are requested again only in this window's second group, after D's last use)
        if constexpr (!Q1) {
          const auto s0 = __builtin_amdgcn_permlane32_swap(W[H][r].x, W[H][r].z, false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(W[H][r].y, W[H][r].w, false, false);
          D[r][0][0] = s0[0];
          D[r][0][1] = s1[0];
          D[r][1][0] = s0[1];
          D[r][1][1] = s1[1];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      ns = cs + 1 < nwin ? cs + 1 : 0;  // the next window's index in its term
      if constexpr (Q1) window_slices(cs, ns);
      pgroup(h_c, FC<0>{});
      __syncthreads();
      pgroup(h_c, FC<1>{});
      cs = ns;
    };
    int w = 0;
    for (; w + 1 < NW; w += 2) {
      pwindow(FC<0>{});
      pwindow(FC<1>{});
    }
    if (w < NW) pwindow(FC<0>{});  // uniform
    // the last group's token tile DT
#pragma unroll
    for (int r = 0; r < F_RT; ++r)
#pragma unroll
      for (int i = 0; i < 4; ++i) total[r][DT][i] += scp[r] * C[r][DT][i];

    // ---- epilogue: lane holds tokens 4 kb + i of each token tile, output row tile_row(wave, r) + r16
    if (glu) {  // (uniform) h = SwiGLU of the lane's gate and up sums, bf16
#pragma unroll
      for (int t = 0; t < TT; ++t) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int tk = 16 * t + 4 * kb + i;
          if (tk >= ntok) continue;
          const int64_t tok = tok0 + tk;
          float w = 1.f;
          if (a.glu_v4 && a.glu_weights) w = a.glu_weights[a.glu_order ? clamp_i64(a.glu_order[tok], 0, a.glu_pairs - 1) : tok];
#pragma unroll
          for (int q = 0; q < 2; ++q) {
            const int64_t col = tile_row(wave, q);
            if (col < 0) continue;
            float g = bf16_bits_to_f32(f32_to_bf16_bits(total[q][t][i])), u = bf16_bits_to_f32(f32_to_bf16_bits(total[q + 2][t][i]));
            float v;
            if (a.glu_v4) {
              if (a.glu_limit > 0.f) {  // torch.clamp: a NaN stays a NaN
                u = u < -a.glu_limit ? -a.glu_limit : (u > a.glu_limit ? a.glu_limit : u);
                g = g > a.glu_limit ? a.glu_limit : g;
              }
              v = (g / (1.0f + expf(-g))) * u;
              if (a.glu_weights) v = w * v;
            } else {
              const float sg = bf16_bits_to_f32(f32_to_bf16_bits(g / (1.0f + expf(-g))));
              v = sg * u;
            }
            a.glu_h[tok * NH + col + r16] = f32_to_bf16_bits(v);
          }
        }
      }
      return;
    }
#pragma unroll
    for (int t = 0; t < TT; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int tk = 16 * t + 4 * kb + i;
        if (tk < ntok) {
          const int64_t tok = tok0 + tk;
#pragma unroll
          for (int r = 0; r < F_RT; ++r) {
            const int64_t row = tile_row(wave, r);
            if (row >= 0) {
              if (a.out16) {
                a.out16[tok * a.N + row + r16] = f32_to_bf16_bits(total[r][t][i]);
              } else {
                float* o = a.out + tok * a.N + row + r16;
                *o = (a.overwrite ? 0.f : *o) + total[r][t][i];
              }
            }
          }
        }
      }
    }
  };
  if (two) all_windows(FC<2>{});
  else all_windows(FC<1>{});
}

template <int SDT, int FMT, int GS>
int launch_gemm_tq2f_g(const GemmArgs& a, hipStream_t s) {
  constexpr int LDS = f_lds_bytes(SDT == BP_F32 ? 4 : 2) + (FMT == BP_TQ1 ? F_LUT + F_WAVES * F_RT * F_TR : 0);
  static_assert(LDS <= 160 * 1024, "LDS of a workgroup");
  const char* name = FMT == BP_TQ1 ? "gemm_tq1f_bf16" : "gemm_tq2f_bf16";
  if (const int rc = raise_lds_limit<k_gemm_tq2f<SDT, FMT, GS>>(LDS)) return rc;
  const int64_t row_blocks = a.glu_h ? (a.N / 2 + F_ROWS / 2 - 1) / (F_ROWS / 2) : (a.N + F_ROWS - 1) / F_ROWS;
  const int64_t wgs = tile_workgroups(a, row_blocks);
  if (wgs < 0) return BP_ERR_UNSUPPORTED;
  const int64_t slots = a.tiles ? a.tile_cap : a.E;
  const unsigned z = a.tiles ? 1u : (unsigned)((a.max_rows + 31) / 32);
  hipLaunchKernelGGL((k_stage_tq2f<FMT == BP_TQ1>), dim3((unsigned)slots, (unsigned)(a.K / 256), z), dim3(F_THREADS), 0, s, a);
  if (const int rc = check_launch("stage_tq2f")) return rc;
  const dim3 grid((unsigned)wgs, 1, 1);
  note_kernel(name);
  hipLaunchKernelGGL((k_gemm_tq2f<SDT, FMT, GS>), grid, dim3(F_THREADS), LDS, s, a);
  return check_launch(name);
}

template <int SDT, int FMT>
int launch_gemm_tq2f_k(const GemmArgs& a, hipStream_t s) {
  return a.group == 256 ? launch_gemm_tq2f_g<SDT, FMT, 1>(a, s) : launch_gemm_tq2f_g<SDT, FMT, 0>(a, s);
}

}  // namespace

// Bytes of workspace the staged path takes for a call with T rows in all, K columns and E experts (0: no staged path
// for these arguments): room for every token tile's windows, tiles placed so that they cannot overlap.
size_t gemm_tq2f_workspace_bytes(int64_t T, int64_t K, int64_t E) {
  if (T <= 0 || K % 256 != 0 || K < 1024 || E <= 0) return 0;
  return (size_t)(T + 32 * E + 32) * (size_t)(K / 256) * (F_FB / 32);
}

// Preconditions (beyond mfma_supports: groups of 128 or 256, K % 256 == 0, K >= 1024, N % 16 == 0, 16-byte aligned x,
// packed rows and scales): a workspace of gemm_tq2f_workspace_bytes in a.stage (16-byte aligned); an even number of
// 16-bit scales per row; bf16 activations (int8 ones have a matrix instruction of their own at twice this one's rate
// per activation: bp_gemm_tq2.hip); offsets into an expert's rows fit 32 bits; a launch whose token tiles mostly exist
// (the conversion runs one workgroup per tile and window: a loose bound on the rows per expert would launch mostly
// empty ones). BP_ERR_UNSUPPORTED (no message): the caller falls back to its other kernels.
int gemm_tq2f_applies(const GemmArgs& a) {
  if (a.x_dtype != BP_BF16 || !a.stage || ((uintptr_t)a.stage & 15) != 0) return BP_ERR_UNSUPPORTED;
  if (a.glu_h && (!a.tiles || !a.overwrite || a.N % 32 != 0)) return BP_ERR_UNSUPPORTED;  // (whole row tiles of either half, one launch for all of K)
  if (a.out16 && (!a.tiles || !a.overwrite)) return BP_ERR_UNSUPPORTED;
  if ((size_t)a.stage_bytes < gemm_tq2f_workspace_bytes(a.T, a.K, a.E) || gemm_tq2f_workspace_bytes(a.T, a.K, a.E) == 0) return BP_ERR_UNSUPPORTED;
  if (a.K > ((int64_t)1 << 24) || a.N * a.Kp > ((int64_t)1 << 31) - 4096) return BP_ERR_UNSUPPORTED;
  if (a.fmt == BP_TQ2 && tuning().tq2g != 'f') {  // (development: BP_TUNE_TQ2G=fp4 runs this kernel wherever it can)
    if (a.N < 2 * F_ROWS) return BP_ERR_UNSUPPORTED;  // (one or two row blocks: converting first saves nothing)
    // One workgroup of 8 waves takes a CU: below three rounds of them (a round = 256 workgroups) the last, partly filled
    // round costs more than the kernel gains over the one that runs two smaller workgroups per CU.
    if ((a.T + 31) / 32 * ((a.N + F_ROWS - 1) / F_ROWS) < 768) return BP_ERR_UNSUPPORTED;
  }
  if (!a.tiles && ((a.max_rows + 31) / 32 > 65535 || (a.max_rows + 31) / 32 * 32 * a.E > 4 * a.T + 32 * a.E)) return BP_ERR_UNSUPPORTED;
  if (a.K / 256 > 65535) return BP_ERR_UNSUPPORTED;
  if (a.group == 256 && a.scale_dtype != BP_F32 && a.G % 2 != 0) return BP_ERR_UNSUPPORTED;  // (rows of scales not dword-aligned)
  if (a.fmt == BP_TQ1) {
    if (a.Kp != (a.K + 4) / 5 || a.scale_dtype == BP_F32) return BP_ERR_UNSUPPORTED;
    for (int t = 1; t < a.n_terms; ++t)  // (one byte alignment of the rows for all terms)
      if ((((uintptr_t)a.packed[t] ^ (uintptr_t)a.packed[0]) & 3) != 0) return BP_ERR_UNSUPPORTED;
  }
  const int64_t row_blocks = a.glu_h ? (a.N / 2 + F_ROWS / 2 - 1) / (F_ROWS / 2) : (a.N + F_ROWS - 1) / F_ROWS;
  if (tile_workgroups(a, row_blocks) < 0) return BP_ERR_UNSUPPORTED;
  return BP_OK;
}

int launch_gemm_tq2f(const GemmArgs& a, hipStream_t s) {
  if (const int rc = gemm_tq2f_applies(a)) return rc;
  if (a.fmt == BP_TQ1) {
    if (a.scale_dtype == BP_F16) return launch_gemm_tq2f_k<BP_F16, BP_TQ1>(a, s);
    return launch_gemm_tq2f_k<BP_BF16, BP_TQ1>(a, s);  // (float32 scales: the table, the transit area and their ring do not fit in LDS together)
  }
  if (a.scale_dtype == BP_F16) return launch_gemm_tq2f_k<BP_F16, BP_TQ2>(a, s);
  if (a.scale_dtype == BP_BF16) return launch_gemm_tq2f_k<BP_BF16, BP_TQ2>(a, s);
  return launch_gemm_tq2f_k<BP_F32, BP_TQ2>(a, s);
}

}  // namespace bp

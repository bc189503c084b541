// Shared pieces of the TQ1 decode GEMV kernels on the fp8 x fp4 matrix instruction (bp_tq1_gemv_fp4.hip,
// bp_tq1_gemv_cw.hip): the byte table, the token's operand A tiles and how a lane finds its blocks in them.
// The scheme is described at the head of bp_tq1_gemv_fp4.hip.
#pragma once
#include <type_traits>

#include "bp_mfma.h"

namespace bp {

// bp_tq1_gemv_cw.hip: the kernel that streams the rows through LDS tile by tile (one token row per expert or a pair,
// rows first_row .. of every expert); BP_ERR_UNSUPPORTED without a message where it does not apply
int launch_tq1_gemv_cw(const GemmArgs& a, hipStream_t s, int ntok, int64_t nchunks, int cus, int first_row);

namespace {

typedef int i32x8 __attribute__((ext_vector_type(8)));
template <int V>
using IC = std::integral_constant<int, V>;
struct __attribute__((packed, aligned(2))) F4Packed16 { u32x4 v; };
struct __attribute__((packed, aligned(2))) F4Packed4 { unsigned v; };

constexpr int F4_LUT_BYTES = 256 * 128;          // byte -> 5 fp4 codes, one copy per bank
// Operand A tile, per chunk: 64 byte pairs x PC pieces x 16 bytes, then 4 group boundaries x PC pieces x 16 bytes, a
// block of zeros, 8 words = the prescales of the chunk's 5 groups (3 unused), 8 floats = their inverses (the unused
// ones are 0): 3344 bytes with 3 pieces, 2256 with 2.
constexpr int f4_pieces(int ntok) { return ntok == 1 ? 3 : 2; }
constexpr int f4_chunk_bytes(int ntok) { return (64 + 4) * f4_pieces(ntok) * 16 + 16 + 32 + 32; }
constexpr int F4_LDS_MAX = 160 * 1024;
// Measured on E = 128, N = 2048, K = 7168: one 16-row tile per wave with 4 chunks in flight reads 504 MB from memory
// per launch, two tiles with 2 chunks each 638 MB (405 MB are packed bytes and scales). Rows of 1434 bytes share
// 128-byte lines between consecutive chunks; the sooner a wave returns to a row, the more of those lines it still
// finds in the L2.
constexpr int F4_SCALE_SLOT = 16 * 80;           // (SR) per wave: 16 rows x 80 bytes (48 of them a round's scales)
constexpr int F4_GR = 1;                         // 16-row tiles per wave (more than one share the reads of operand A)
constexpr int F4_RD = 4;                         // chunks of packed bytes in registers per tile (the ring of loads in flight)
constexpr int F4_BD = 1;                         // table reads run this many (instruction, tile) pairs ahead of the matrix instructions
constexpr int F4_PAIRS = 1;                      // 1: chunks are refilled two at a time (RD even)
constexpr int F4_AD = 0;                         // 1: operand A is read one instruction ahead into a second set of registers

__device__ __forceinline__ u32x2 f4_load8(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned wave_off) {
  return __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)lane_off, (int)wave_off, 0));
}

// first packed byte (of the chunk's 128) of the byte pair behind half `hf` of A lane quarter `kbA` in instruction j.
// MAP 0: B lane (n, kb) brings dword j % 4 of the 16-byte quarter kb of the 64-byte window j / 4 (the bytes as a lane
// loaded them). MAP 1: it brings dword kb of the chunk's 16-byte piece j, so an instruction covers 80 consecutive
// digits - at most two scale groups (the streaming kernel with four token rows per expert).
template <int MAP = 0>
__device__ __forceinline__ int f4_pair_byte(int j, int kbA, int hf) {
  if (MAP == 1) return 16 * j + 4 * (2 * hf + (kbA >> 1)) + 2 * (kbA & 1);
  return 64 * (j >> 2) + 16 * (2 * hf + (kbA >> 1)) + 4 * (j & 3) + 2 * (kbA & 1);
}

// Layout of one chunk of an operand A tile for PC pieces per activation (byte offsets within the chunk's part).
template <int PC>
struct F4Tile {
  static constexpr int HI_OFF = 64 * PC * 16, ZERO_OFF = HI_OFF + 4 * PC * 16, PRE_OFF = ZERO_OFF + 16;
  static constexpr int INV_OFF = PRE_OFF + 32, CHUNK_BYTES = (64 + 4) * PC * 16 + 16 + 32 + 32;
};

// ---- the byte table: entry v = digits d0..d4 of v as fp4 codes (-1 -> 0xA, 0 -> 0, +1 -> 0x2) in nibbles 0..4, one
// copy per LDS bank: four threads per entry, eight copies each.
template <int THREADS>
__device__ __forceinline__ void f4_build_table() {
  for (int idx = threadIdx.x; idx < 256 * 4; idx += THREADS) {
    unsigned v = (unsigned)idx >> 2, ent = 0;
    if (v < 243) {
#pragma unroll
      for (int d = 0; d < 5; ++d) {
        const unsigned q = v / 3, dig = v - 3 * q;
        ent |= (dig == 0 ? 0xAu : dig == 2 ? 0x2u : 0u) << (4 * d);
        v = q;
      }
    }
#pragma unroll
    for (int cpy = 0; cpy < 8; ++cpy) *(lds_u32*)(128 * (idx >> 2) + 4 * (8 * (idx & 3) + cpy)) = ent;
  }
}

// The operand A tiles of the launch's `ntok` tokens (rows tok, tok + 1, ... of x) for chunks cb .. cb + nchunks - 1, built
// behind the table (from LDS byte AT) by the workgroup's first `builders` waves (the caller synchronises afterwards).
struct F4Nothing { __device__ __forceinline__ void operator()() const {} };
// `meanwhile` runs after the wave's first activations are requested and before they are used.
template <int NTOK, int WAVES, int AT = F4_LUT_BYTES, int MAP = 0, typename Meanwhile = F4Nothing>
__device__ __forceinline__ void f4_build_tiles(const GemmArgs& a, int64_t tok, int ntok, int nchunks, int cb, int wave, int lane, int builders = WAVES, Meanwhile meanwhile = Meanwhile()) {
  constexpr int PC = f4_pieces(NTOK);
  constexpr int F4_HI_OFF = F4Tile<PC>::HI_OFF, F4_ZERO_OFF = F4Tile<PC>::ZERO_OFF, F4_PRE_OFF = F4Tile<PC>::PRE_OFF;
  constexpr int F4_INV_OFF = F4Tile<PC>::INV_OFF, F4_CHUNK_BYTES = F4Tile<PC>::CHUNK_BYTES;
  auto tile_at = [](int tt, int c) { return AT + (c * NTOK + tt) * F4_CHUNK_BYTES; };
  const bool x16 = a.x_dtype == BP_BF16 || a.x_dtype == BP_F16;
  auto widen16 = [&](unsigned h) { return a.x_dtype == BP_BF16 ? bf16_bits_to_f32((uint16_t)h) : f16_bits_to_f32((uint16_t)h); };
  // ---- operand A tiles: a wave builds whole chunks by itself (64 byte pairs = 64 lanes; a chunk holds 5 whole scale
  // groups), so the activations are read from memory once and nothing waits for another wave until the tiles are
  // complete. Lane = byte pair: its 10 activations -> the largest magnitude of each of its (one or two) groups by an LDS
  // maximum over the float bits -> the groups' prescales 2^sh (sh brings the group's largest magnitude into [128, 256))
  // and their inverses -> 3 pieces x (first-group block, second-group block).
  const int blk = lane;
  const int tt0 = 5 * f4_pair_byte<MAP>(blk >> 3, (blk >> 1) & 3, blk & 1), glo = tt0 >> 7, ghi = (tt0 + 9) >> 7;
  // (a wave with several items requests the next item's activations before it works on the current one's)
  // The lane's 10 activations come as one 20-byte piece (16-bit) or as the three dwords around their 10 bytes (int8)
  // through a buffer over the whole tensor: what lies past it reads as zero, what lies past the row is masked below.
  const int esz = x16 ? 2 : 1;
  const bool vec = a.x_dtype != BP_F32 && ((uintptr_t)a.x & 3) == 0 && a.T * a.K * esz < 0x7ffffff0 && (!x16 || (a.K & 1) == 0);
  const __amdgpu_buffer_rsrc_t xrs = make_rsrc(a.x, whole_dwords(a.T * a.K * esz));
  u32x4 qn = {0u, 0u, 0u, 0u};
  unsigned q4n = 0u, xsn = 0u;
  auto request_x = [&](int item) {
    const int tt = item / nchunks, c = item - tt * nchunks;
    const int64_t k0 = 640 * (int64_t)(cb + c) + tt0;
    if (vec && item < ntok * nchunks) {
      const unsigned bo = (unsigned)(((tok + tt) * a.K + k0) * esz);
      if (x16) {
        qn = buf_load16(xrs, bo, 0u);
        q4n = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(xrs, (int)(bo + 16u), 0, 0);
      } else {
        const u32x2 lo = f4_load8(xrs, bo & ~3u, 0u);
        qn = u32x4{lo.x, lo.y, (unsigned)__builtin_amdgcn_raw_buffer_load_b32(xrs, (int)((bo & ~3u) + 8u), 0, 0), 0u};
        xsn = bo & 3u;
      }
    }
  };
  request_x(wave);
  meanwhile();
  for (int item = wave; item < ntok * nchunks; item += builders) {  // (the waves 0 .. builders - 1 call this)
    const int tt = item / nchunks, c = item - tt * nchunks;
    const int64_t xrow = (tok + tt) * a.K;
    const unsigned dst = (unsigned)tile_at(tt, c);
    if (lane < 8) *(lds_u32*)(dst + F4_PRE_OFF + 4 * lane) = 0u;
    const int64_t k0 = 640 * (int64_t)(cb + c) + tt0;
    float y[10];
    const u32x4 q = qn;
    const unsigned q4 = q4n, xs = xsn;
    request_x(item + builders);
    if (vec && x16) {
#pragma unroll
      for (int i = 0; i < 4; ++i) { y[2 * i] = widen16(q[i] & 0xffffu); y[2 * i + 1] = widen16(q[i] >> 16); }
      y[8] = widen16(q4 & 0xffffu);
      y[9] = widen16(q4 >> 16);
    } else if (vec) {
      const unsigned d[3] = {__builtin_amdgcn_alignbyte(q.y, q.x, xs), __builtin_amdgcn_alignbyte(q.z, q.y, xs), __builtin_amdgcn_alignbyte(0u, q.z, xs)};
#pragma unroll
      for (int t = 0; t < 10; ++t) y[t] = (float)(int)(int8_t)((d[t >> 2] >> (8 * (t & 3))) & 0xffu);
    }
    if (vec) {
      if (640 * (int64_t)(cb + c + 1) > a.K) {  // (uniform: the row's last chunk)
#pragma unroll
        for (int t = 0; t < 10; ++t) y[t] = k0 + t < a.K ? y[t] : 0.f;
      }
    } else {
#pragma unroll
      for (int t = 0; t < 10; ++t) y[t] = k0 + t < a.K ? load_act_f32(a.x, a.x_dtype, xrow + k0 + t) : 0.f;
    }
    if (a.x_dtype != BP_I8) {  // (int8 values fit as they are: prescale 1)
      unsigned m_lo = 0, m_hi = 0;
#pragma unroll
      for (int t = 0; t < 10; ++t) {
        const unsigned v = __float_as_uint(y[t]) & 0x7fffffffu;
        if (((tt0 + t) >> 7) == glo) m_lo = m_lo > v ? m_lo : v;
        else m_hi = m_hi > v ? m_hi : v;
      }
      __hip_atomic_fetch_max((lds_u32*)(dst + F4_PRE_OFF + 4 * glo), m_lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
      if (ghi != glo) __hip_atomic_fetch_max((lds_u32*)(dst + F4_PRE_OFF + 4 * ghi), m_hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (lane < 8) {
      const int g = lane;
      const unsigned at = dst + 4 * g;
      const bool real = g < 5 && 128 * (int64_t)(5 * (cb + c) + g) < a.K;
      int sh = 0;
      bool finite = true;
      if (real && a.x_dtype != BP_I8) {
        const int ex = (int)((*(const lds_u32*)(at + F4_PRE_OFF) >> 23) & 255u);
        finite = ex != 255;  // a NaN or an infinity among the group's activations
        sh = 134 - ex;
        sh = sh > 120 ? 120 : sh < -120 ? -120 : sh;
      }
      *(lds_u32*)(at + F4_PRE_OFF) = (unsigned)(sh + 127) << 23;
      // (the inverse prescale multiplies every row's group sum: NaN for a group with a non-finite activation, so the
      // token's outputs are NaN rather than finite and wrong)
      *(lds_u32*)(at + F4_INV_OFF) = !real ? 0u : finite ? (unsigned)(127 - sh) << 23 : 0x7fc00000u;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float pre_lo = __uint_as_float(*(const lds_u32*)(dst + F4_PRE_OFF + 4 * glo));
    const float pre_hi = __uint_as_float(*(const lds_u32*)(dst + F4_PRE_OFF + 4 * ghi));
    u32x4 lo[PC] = {}, hi[PC] = {};
#pragma unroll
    for (int t = 0; t < 10; t += 2) {  // two activations per conversion
      const bool in0 = ((tt0 + t) >> 7) == glo, in1 = ((tt0 + t + 1) >> 7) == glo;
      float r0 = y[t] * (in0 ? pre_lo : pre_hi), r1 = y[t + 1] * (in1 ? pre_lo : pre_hi);
      const int pos0 = 8 * (t / 5) + t % 5, pos1 = 8 * ((t + 1) / 5) + (t + 1) % 5;  // digit slots of the block
#pragma unroll
      for (int p = 0; p < PC; ++p) {
        const int w = __builtin_amdgcn_cvt_pk_fp8_f32(p == 2 ? r0 * 256.f : r0, p == 2 ? r1 * 256.f : r1, 0, false);
        if (p + 1 < PC) {
          r0 -= __builtin_amdgcn_cvt_f32_fp8(w, 0);
          r1 -= __builtin_amdgcn_cvt_f32_fp8(w, 1);
        }
        const unsigned c0 = (unsigned)w & 0xffu, c1 = ((unsigned)w >> 8) & 0xffu;
        lo[p][pos0 >> 2] |= (in0 ? c0 : 0u) << (8 * (pos0 & 3));
        hi[p][pos0 >> 2] |= (in0 ? 0u : c0) << (8 * (pos0 & 3));
        lo[p][pos1 >> 2] |= (in1 ? c1 : 0u) << (8 * (pos1 & 3));
        hi[p][pos1 >> 2] |= (in1 ? 0u : c1) << (8 * (pos1 & 3));
      }
    }
#pragma unroll
    for (int p = 0; p < PC; ++p) *(lds_u32x4*)(dst + 16 * (PC * blk + p)) = lo[p];
    if (ghi != glo) {
#pragma unroll
      for (int p = 0; p < PC; ++p) *(lds_u32x4*)(dst + F4_HI_OFF + 16 * (PC * (ghi - 1) + p)) = hi[p];
    }
    if (blk == 0) *(lds_u32x4*)(dst + F4_ZERO_OFF) = u32x4{0u, 0u, 0u, 0u};
  }
}

// A lane as a row of operand A (rows 4 g + p = piece p of group g < 4; rows 3, 7, 11 = pieces of group 4; row 15 unused;
// several tokens: row 4 s + 2 t + p = piece p of the pair's token t in group slot s < 3, rows 12..15 unused): the 16-byte
// block (index within the chunk's part of the tile) of instruction j, half hf, in byte 2 (j % 2) + hf of aoff[j / 2].
template <int PC>
__device__ __forceinline__ void f4_block_offsets(int r16, int kb, unsigned (&aoff)[4]) {
  constexpr int F4_HI_OFF = F4Tile<PC>::HI_OFF, F4_ZERO_OFF = F4Tile<PC>::ZERO_OFF;
  const int am_g = PC == 2 ? r16 >> 2 : (r16 & 3) < 3 ? r16 >> 2 : 4, am_p = PC == 2 ? r16 & 1 : (r16 & 3) < 3 ? r16 & 3 : r16 >> 2;
  const bool am_used = PC == 2 ? r16 < 12 : r16 < 15;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    unsigned both = 0;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int blk = j * 8 + kb * 2 + hf;
      const int tt0 = 5 * f4_pair_byte(j, kb, hf), glo = tt0 >> 7, ghi = (tt0 + 9) >> 7;
      // (several tokens: the group behind the lane's slot in this instruction's window)
      const int g = PC == 3 || j < 4 ? am_g : am_g == 0 ? 3 : am_g == 1 ? 4 : 2;
      unsigned o = F4_ZERO_OFF / 16;
      if (am_used && g == glo) o = PC * blk + am_p;
      else if (am_used && g == ghi) o = F4_HI_OFF / 16 + PC * (ghi - 1) + am_p;
      both |= o << (8 * hf);
    }
    if (j & 1) aoff[j >> 1] |= both << 16;
    else aoff[j >> 1] = both;
  }
}

// Four token rows per expert over byte map 1: row 8 s + 2 t + p = piece p of token t (which selects the token's tile, not
// the block) in group slot s, and slot s of an instruction holds the group of its 80 digits whose number has parity s.
// An accumulator tile may collect instructions as long as neither slot changes its group: instructions 0-2 (groups 0 | 1),
// 3 (2 | 1), 4-5 (2 | 3), 6-7 (4 | 3).
__device__ __forceinline__ void f4_block_offsets4(int r16, int kb, unsigned (&aoff)[4]) {
  constexpr int PC = 2, F4_HI_OFF = F4Tile<PC>::HI_OFF, F4_ZERO_OFF = F4Tile<PC>::ZERO_OFF;
  const int am_s = r16 >> 3, am_p = r16 & 1;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    unsigned both = 0;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int blk = j * 8 + kb * 2 + hf;
      const int tt0 = 5 * f4_pair_byte<1>(j, kb, hf), glo = tt0 >> 7, ghi = (tt0 + 9) >> 7;
      unsigned o = F4_ZERO_OFF / 16;
      if ((glo & 1) == am_s) o = PC * blk + am_p;
      else if (ghi != glo) o = F4_HI_OFF / 16 + PC * (ghi - 1) + am_p;
      both |= o << (8 * hf);
    }
    if (j & 1) aoff[j >> 1] |= both << 16;
    else aoff[j >> 1] = both;
  }
}

inline int f4_cus() {  // compute units of the current device (256 if the query fails); looked up once per device
  static std::mutex m;
  static int known[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  std::lock_guard<std::mutex> lock(m);
  if (known[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) cus = 256;
    known[dev] = cus;
  }
  return known[dev];
}

}  // namespace
}  // namespace bp

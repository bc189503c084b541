// TQ2 (4 trits per byte) decode into MFMA operands, shared by the TQ2 kernels.
#pragma once
#include "bp_mfma.h"

namespace bp {
namespace {

// ---- TQ2 decode without a table.
// bf16: a 2-bit code u placed at bits [7:6] of a bf16 whose other bits are 0x4000 reads 2 + u (the code
// spans the lowest exponent bit and the highest mantissa bit: 2, 3, 4); placed at bits [5:4] of 0x4100 it
// reads 8 + u. One v_and_or_b32 per output dword therefore turns two codes of a packed dword (one per
// 16-bit half) into two bf16 values; three shifts bring all 16 codes of the dword to those two positions.
// The products then carry sum(x * (c + u)) with c = 2 (odd trits) or 8 (even trits); the accumulator of
// every group starts from -sum(x * (c + 1)), computed once per workgroup when the activation tile is
// staged, which leaves sum(x * (u - 1)). Slot order of the two operands made from a packed dword (codes
// c0..c15, lo/hi bf16 of each operand dword):
//   first  : (c3,c11) (c2,c10) (c1,c9) (c0,c8)      second : (c5,c13) (c4,c12) (c7,c15) (c6,c14)
// The activation tile is stored in LDS in that order (permuted inside every 16 elements when staged).
// The unused code 3 reads +3 or +2 depending on its slot (pack never writes it).
struct Tq2Consts { unsigned P1, P2, M1, M2; };  // 0x00c000c0, 0x00300030, 0x40004000, 0x41004100 held in registers
__device__ __forceinline__ void tq2_decode_bf16(unsigned w, const Tq2Consts& k, u32x4& first, u32x4& second) {
  const unsigned P1 = k.P1, P2 = k.P2, M1 = k.M1, M2 = k.M2;
  const unsigned wl = w << 4, wr = w >> 4, wr8 = w >> 8;
  first = u32x4{(w & P1) | M1, (w & P2) | M2, (wl & P1) | M1, (wl & P2) | M2};
  second = u32x4{(wr & P1) | M1, (wr & P2) | M2, (wr8 & P1) | M1, (wr8 & P2) | M2};
}
// int8: dword i of the operand = codes c(i), c(i+4), c(i+8), c(i+12) as digits 0..2; the accumulator
// starts from -sum(x). The activation tile is stored with every 16 bytes transposed 4 x 4 to match.
__device__ __forceinline__ u32x4 tq2_decode_i8(unsigned w) {
  const unsigned m = 0x03030303u;
  return u32x4{w & m, (w >> 2) & m, (w >> 4) & m, (w >> 6) & m};
}
__device__ __forceinline__ void tq2_permute_bf16(const u32x4 a, const u32x4 c, u32x4& o0, u32x4& o1) {
  const unsigned HI = 0x07060302u, LO = 0x05040100u;
  o0 = u32x4{__builtin_amdgcn_perm(c.y, a.y, HI), __builtin_amdgcn_perm(c.y, a.y, LO),
             __builtin_amdgcn_perm(c.x, a.x, HI), __builtin_amdgcn_perm(c.x, a.x, LO)};
  o1 = u32x4{__builtin_amdgcn_perm(c.z, a.z, HI), __builtin_amdgcn_perm(c.z, a.z, LO),
             __builtin_amdgcn_perm(c.w, a.w, HI), __builtin_amdgcn_perm(c.w, a.w, LO)};
}
__device__ __forceinline__ u32x4 tq2_permute_i8(const u32x4 a) {
  const unsigned s0 = __builtin_amdgcn_perm(a.y, a.x, 0x05010400u), s1 = __builtin_amdgcn_perm(a.y, a.x, 0x07030602u);
  const unsigned s2 = __builtin_amdgcn_perm(a.w, a.z, 0x05010400u), s3 = __builtin_amdgcn_perm(a.w, a.z, 0x07030602u);
  return u32x4{__builtin_amdgcn_perm(s2, s0, 0x05040100u), __builtin_amdgcn_perm(s2, s0, 0x07060302u),
               __builtin_amdgcn_perm(s3, s1, 0x05040100u), __builtin_amdgcn_perm(s3, s1, 0x07060302u)};
}

}  // namespace
}  // namespace bp

// Shared pieces of the tuned gfx950 MFMA kernels (bp_mfma_tq2.hip, bp_mfma_tq1.hip).
//
// Packed trits are decoded in registers straight into MFMA operands, one 16-row x 16-token tile per
// instruction (v_mfma_f32_16x16x32_bf16 for bf16 activations, v_mfma_i32_16x16x64_i8 for int8).
// Accumulators are flushed at every 128-wide K group: total += acc * scale[n, g] in float32, so the
// scale multiplies the group sum exactly as in the reference contract
// (boilerplate/kernels/ternary_cuda.py:58-63, boilerplate/kernels/csrc/boilerplate_cpu.cpp:114-124).
// Stacked terms share one staging of the activations and one output write.
//
// Operand A = activations (row i = token), operand B = weights (column j = output row), so a lane
// ends with 4 tokens x 1 output row and needs one scale per group.
//
// The kernels address LDS absolutely: they declare no static LDS, so the dynamic allocation requested
// at launch starts at LDS address 0.
#pragma once
#include <cstdlib>

#include "bp_common.h"

namespace bp {

// implemented in bp_mfma_tq2.hip / bp_mfma_tq1.hip; R, MT, waves: the tiling chosen by launch_mfma
int launch_mfma_tq2(const GemmArgs& a, hipStream_t s, int R, int MT, int waves);
int launch_mfma_tq1(const GemmArgs& a, hipStream_t s, int waves);
// bp_gemm_tq2.hip: TQ2 with token tiles of 32 (experts with more than 16 token rows)
int launch_gemm_tq2(const GemmArgs& a, hipStream_t s);
int launch_gemm_tq2f(const GemmArgs& a, hipStream_t s);
int gemm_tq2f_applies(const GemmArgs& a);  // BP_OK where launch_gemm_tq2f takes the call (nothing is launched)
// bp_gemm_tq1.hip: TQ1 with token tiles of 32 on the fp8 x fp4 matrix instruction (experts with more than 8 token rows);
// BP_ERR_UNSUPPORTED without a message when the call is outside its preconditions
int launch_gemm_tq1(const GemmArgs& a, hipStream_t s);
// TQ1 calls of seven or eight token rows per expert that run on the tile kernel over converted activations when the
// caller brings a workspace, rather than as two launches of the four-row decode kernel: dense batches (four rows per
// expert on average) of at least 512 blocks of 512 output rows. Measured with 8 rows per expert: 128 experts x 2048 x
// 7168 204 against 230 us, 64 x 4096 x 4096 113 against 130 us, 128 x 7168 x 2048 268 against 272 us; 16 experts x
// 2048 x 7168 (64 blocks) 82 against 79 us; six rows per expert 203 against 198 us.
inline bool tq1_rows_on_tiles(int64_t max_rows, int64_t E, int64_t T, int64_t N) {
  return max_rows >= 7 && max_rows <= 8 && T >= 4 * E && (E < T ? E : T) * ((N + 511) / 512) >= 512;
}
// bp_tq1_gemv.hip: TQ1, one token row per expert (max_rows == 1), bf16 activations, table-lookup GEMV
int launch_tq1_gemv(const GemmArgs& a, hipStream_t s, int waves);
// bp_tq1_gemv_fp4.hip: the same through the fp8 x fp4 matrix instruction (16-bit and int8 activations), and small
// batches: up to 8 token rows per expert, or up to 64 in launches of 8 when the experts average at most 4 rows;
// BP_ERR_UNSUPPORTED without a message when the call is outside its preconditions
int launch_tq1_gemv_fp4(const GemmArgs& a, hipStream_t s);
// bp_tq2_gemv_fp4.hip: TQ2, one to four token rows per expert, on the fp8 x fp4 matrix instruction with K split over the waves;
// BP_ERR_UNSUPPORTED without a message when the call is outside its preconditions
int launch_tq2_gemv_fp4(const GemmArgs& a, hipStream_t s);

namespace {

typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) u32x2 lds_u32x2;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) unsigned lds_u32;
typedef __attribute__((address_space(3))) unsigned short lds_u16;

// Weights and scales are read with raw buffer loads: a wave-uniform descriptor (base, byte range) in
// scalar registers, a 32-bit lane offset and a scalar step offset, so a load needs no vector address
// arithmetic, and a read past the range returns zeros instead of touching memory.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int64_t bytes) {
  const int n = bytes > 0x7fffffff ? 0x7fffffff : (int)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), (short)0, n, 0x00020000);
}
// A buffer load returns zero for a dword that straddles the end of its range, valid bytes included. Ranges over tensors
// that may start at any byte (the base is aligned down to a dword by the caller) therefore end with the dword that holds
// the tensor's last byte: up to 3 bytes behind the tensor are read with it - inside a dword of which the tensor owns a
// byte - and never used.
__device__ __forceinline__ int64_t whole_dwords(int64_t bytes) { return (bytes + 3) & ~(int64_t)3; }
__device__ __forceinline__ u32x4 buf_load16(__amdgpu_buffer_rsrc_t r, unsigned lane_off, unsigned wave_off) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_off, (int)wave_off, 0));
}

template <int ACT>
struct Acc;
template <>
struct Acc<BP_BF16> { typedef f32x4 type; };
template <>
struct Acc<BP_I8> { typedef i32x4 type; };

template <int SDT>
__device__ __forceinline__ float scale_at(const u32x4 (&raw)[2], int i) {  // i-th of the 8 scales held in raw
  if (SDT == BP_F32) return __uint_as_float(raw[i >> 2][i & 3]);
  const unsigned v = raw[i >> 3][(i >> 1) & 3];
  if (SDT == BP_F16) return f16_bits_to_f32((uint16_t)((i & 1) ? (v >> 16) : (v & 0xffffu)));
  return __uint_as_float((i & 1) ? (v & 0xffff0000u) : (v << 16));
}

}  // namespace
}  // namespace bp

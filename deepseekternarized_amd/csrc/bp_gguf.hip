// Boilerplate single-term ternary weights <-> llama.cpp's TQ1_0 / TQ2_0 blocks (GGUF interop).
//
// The reference converts a Mode C / D weight with one term, group 256 and fp16 scales by dequantizing it and handing the
// values to `gguf.quants.quantize` (boilerplate/format/gguf_export.py:45-58 `_single_term`, :103-114 `quantize_exact`),
// then checks that the blocks dequantize back to the same values bit for bit. These kernels produce the same blocks
// straight from the packed rows, and read such blocks back into trits and scales.
//
// Block layouts (llama.cpp ggml/src/ggml-common.h; 256 weights per block, one fp16 scale d):
//   TQ2_0, 66 bytes: qs[64], d. Two chunks of 128 weights; byte m of a chunk holds weights m, m + 32, m + 64, m + 96 of
//          the chunk as 2-bit digits (trit + 1) at bits 0, 2, 4, 6.
//   TQ1_0, 54 bytes: qs[48], qh[4], d. qs[0..31]: byte m holds weights m + 32 n (n = 0..4) of the first 160; qs[32..47]:
//          byte 32 + m holds weights 160 + m + 16 n of the next 80; qh[j]: weights 240 + j + 4 n (n = 0..3). A byte is
//          q = sum digit_n 3^(4 - n) (first weight most significant; qh: times 3) stored as ceil(256 q / 243), so that
//          digit n reads back as (((byte * 3^n) mod 256) * 3) >> 8.
// quantize_row_tq{1,2}_0_ref (ggml/src/ggml-quants.c): d = max |x| of the block, digit = lroundf(x * (1 / d)) + 1 (d = 0:
// every digit 1), d stored as fp16.
#include "bp_common.h"

namespace bp {
namespace {

__device__ __forceinline__ int ternary_at(const uint8_t* row, int64_t k, int fmt) {  // boilerplate/ternary/pack.py:48-51, 73-74
  if (fmt == BP_TQ2) return (int)((row[k >> 2] >> (2 * (k & 3))) & 3) - 1;
  return tq1_trit(row[k / 5], (int)(k % 5));
}

__device__ __forceinline__ unsigned tq1_0_byte(const int* dig, int n, int stride) {  // n digits, most significant first
  int q = 0;
  for (int i = 0; i < n; ++i) q = q * 3 + dig[i * stride];
  if (n == 4) q *= 3;
  return (unsigned)((q * 256 + 242) / 243);
}

// One wave per (row, block of 256 weights), four waves per workgroup: lane l holds weights l, l + 64, l + 128, l + 192 of
// the block; the digits cross lanes through the wave's own 256 entries of LDS (no workgroup barrier: a wave's LDS
// accesses complete in order).
constexpr int GGUF_WAVES = 4;
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int QT>
__global__ __launch_bounds__(64 * GGUF_WAVES) void k_gguf_from_ternary(uint8_t* __restrict__ blocks, const uint8_t* __restrict__ packed,
                                                                       const uint16_t* __restrict__ scale, int64_t Kp, int64_t nb, int64_t total,
                                                                       int fmt) {
  constexpr int BS = QT == BP_GGUF_TQ1_0 ? 54 : 66;
  __shared__ int dig_all[GGUF_WAVES][256];
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t blk = (int64_t)blockIdx.x * GGUF_WAVES + wv;
  if (blk >= total) return;  // (uniform for the wave)
  const int64_t n = blk / nb, b = blk - n * nb;
  int* dig = dig_all[wv];
  const float s = f16_bits_to_f32(scale[blk]);
  float v[4], m = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    v[j] = (float)ternary_at(packed + n * Kp, 256 * b + lane + 64 * j, fmt) * s;
    m = fmaxf(m, fabsf(v[j]));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  const float d = m;
  const float id = d != 0.f ? 1.0f / d : 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) dig[lane + 64 * j] = (int)lroundf(v[j] * id) + 1;
  wave_lds_sync();
  uint8_t* out = blocks + blk * BS;
  const int t = lane;
  if (QT == BP_GGUF_TQ2_0) {
    const int* c = dig + 128 * (t >> 5) + (t & 31);
    out[t] = (uint8_t)((c[0] & 3) | ((c[32] & 3) << 2) | ((c[64] & 3) << 4) | ((c[96] & 3) << 6));
  } else {
    if (t < 32) out[t] = (uint8_t)tq1_0_byte(dig + t, 5, 32);
    else if (t < 48) out[t] = (uint8_t)tq1_0_byte(dig + 160 + (t - 32), 5, 16);
    else if (t < 52) out[t] = (uint8_t)tq1_0_byte(dig + 240 + (t - 48), 4, 4);
  }
  if (t == 63) {
    const _Float16 h = (_Float16)d;  // round to nearest even, as GGML_FP32_TO_FP16
    const uint16_t bits = __builtin_bit_cast(uint16_t, h);
    out[BS - 2] = (uint8_t)(bits & 0xff);
    out[BS - 1] = (uint8_t)(bits >> 8);
  }
}

template <int QT>
__global__ __launch_bounds__(64 * GGUF_WAVES) void k_gguf_to_trits(int8_t* __restrict__ trits, uint16_t* __restrict__ scale,
                                                                   const uint8_t* __restrict__ blocks, int64_t K, int64_t nb, int64_t total) {
  constexpr int BS = QT == BP_GGUF_TQ1_0 ? 54 : 66;
  const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t blk = (int64_t)blockIdx.x * GGUF_WAVES + wv;
  if (blk >= total) return;
  const int64_t n = blk / nb, b = blk - n * nb;
  const uint8_t* in = blocks + blk * BS;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int t = lane + 64 * j;
    int digit;
    if (QT == BP_GGUF_TQ2_0) {
      digit = (in[32 * (t >> 7) + (t & 31)] >> (2 * ((t >> 5) & 3))) & 3;
    } else {
      unsigned byte, i;
      if (t < 160) { byte = in[t & 31]; i = (unsigned)t >> 5; }
      else if (t < 240) { byte = in[32 + ((t - 160) & 15)]; i = (unsigned)(t - 160) >> 4; }
      else { byte = in[48 + ((t - 240) & 3)]; i = (unsigned)(t - 240) >> 2; }
      const unsigned p3 = i == 0 ? 1u : i == 1 ? 3u : i == 2 ? 9u : i == 3 ? 27u : 81u;
      digit = (int)((((byte * p3) & 0xffu) * 3u) >> 8);
    }
    trits[n * K + 256 * b + t] = (int8_t)(digit - 1);
  }
  if (lane == 0) scale[blk] = (uint16_t)(in[BS - 2] | ((unsigned)in[BS - 1] << 8));
}

}  // namespace
}  // namespace bp

using namespace bp;

static int gguf_dims(int64_t N, int64_t K, int qtype) {
  if (qtype != BP_GGUF_TQ1_0 && qtype != BP_GGUF_TQ2_0) return fail(BP_ERR_ARG, "qtype must be BP_GGUF_TQ1_0 or BP_GGUF_TQ2_0");
  if (N < 0 || K <= 0 || K % 256 != 0 || N > 65535 || K / 256 > 0x7fffffff / 16384)  // (N K / 1024 workgroups in one grid dimension)
    return fail(BP_ERR_ARG, "ggml TQ blocks hold 256 weights: K must be a multiple of 256 (and N at most 65535 rows per call)");
  return BP_OK;
}

extern "C" int64_t bp_gguf_block_bytes(int qtype) { return qtype == BP_GGUF_TQ1_0 ? 54 : qtype == BP_GGUF_TQ2_0 ? 66 : 0; }

extern "C" int bp_gguf_from_ternary(uint8_t* blocks, int qtype, const uint8_t* packed, const void* scale, int64_t N, int64_t K,
                                    int fmt, void* stream) {
  if (const int rc = gguf_dims(N, K, qtype)) return rc;
  if (fmt != BP_TQ1 && fmt != BP_TQ2) return fail(BP_ERR_ARG, "fmt must be 1 (TQ1) or 2 (TQ2)");
  if (N == 0) return BP_OK;
  if (!blocks || !packed || !scale) return fail(BP_ERR_ARG, "null pointer");
  const int64_t Kp = fmt == BP_TQ2 ? (K + 3) / 4 : (K + 4) / 5, nb = K / 256;
  const int64_t total = N * nb;
  const dim3 grid((unsigned)((total + GGUF_WAVES - 1) / GGUF_WAVES));
  if (qtype == BP_GGUF_TQ1_0) hipLaunchKernelGGL(k_gguf_from_ternary<BP_GGUF_TQ1_0>, grid, dim3(64 * GGUF_WAVES), 0, (hipStream_t)stream, blocks, packed, (const uint16_t*)scale, Kp, nb, total, fmt);
  else hipLaunchKernelGGL(k_gguf_from_ternary<BP_GGUF_TQ2_0>, grid, dim3(64 * GGUF_WAVES), 0, (hipStream_t)stream, blocks, packed, (const uint16_t*)scale, Kp, nb, total, fmt);
  return check_launch("gguf_from_ternary");
}

extern "C" int bp_gguf_to_trits(int8_t* trits, void* scale, const uint8_t* blocks, int qtype, int64_t N, int64_t K, void* stream) {
  if (const int rc = gguf_dims(N, K, qtype)) return rc;
  if (N == 0) return BP_OK;
  if (!trits || !scale || !blocks) return fail(BP_ERR_ARG, "null pointer");
  const int64_t nb = K / 256;
  const int64_t total = N * nb;
  const dim3 grid((unsigned)((total + GGUF_WAVES - 1) / GGUF_WAVES));
  if (qtype == BP_GGUF_TQ1_0) hipLaunchKernelGGL(k_gguf_to_trits<BP_GGUF_TQ1_0>, grid, dim3(64 * GGUF_WAVES), 0, (hipStream_t)stream, trits, (uint16_t*)scale, blocks, K, nb, total);
  else hipLaunchKernelGGL(k_gguf_to_trits<BP_GGUF_TQ2_0>, grid, dim3(64 * GGUF_WAVES), 0, (hipStream_t)stream, trits, (uint16_t*)scale, blocks, K, nb, total);
  return check_launch("gguf_to_trits");
}

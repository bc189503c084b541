// General-shape kernels: the any-K / any-group ternary GEMM and the elementwise format kernels
// (unpack, pack, scale expansion, TQ1 table, int8 activation quantisation).
//
// The general GEMM follows the arithmetic of the reference contract literally
// (boilerplate/kernels/ternary_cuda.py:52-64): exact int32 group sums, then in float32
// y += float(acc) * scale[g] with the multiply and the add rounded separately, in ascending group
// order, then y * x_scale. One wavefront owns one output row n of one expert and up to TOK token
// rows; the 64 lanes stride over the k of a group and the group sum is reduced across the wave.
#include "bp_common.h"

namespace bp {
namespace {

constexpr int GEN_WAVES = 4;  // output rows per workgroup
constexpr int GEN_TOK = 4;    // token rows per pass

__device__ __forceinline__ int decode_trit(const uint8_t* row, int64_t k, int fmt, const int8_t* lut) {
  if (fmt == BP_TQ2) {
    const unsigned b = row[k >> 2];
    return (int)((b >> ((k & 3) * 2)) & 3u) - 1;
  }
  const unsigned b = row[k / 5];
  return lut[b * 5 + (int)(k % 5)];
}

template <bool INT8>
__global__ __launch_bounds__(GEN_WAVES * 64) void k_general(GemmArgs a) {
  __shared__ int8_t lut[256 * 5];
  for (int i = threadIdx.x; i < 256 * 5; i += blockDim.x) lut[i] = (int8_t)tq1_trit(i / 5, i % 5);
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t e = blockIdx.y;
  const int64_t n = (int64_t)blockIdx.x * GEN_WAVES + wave;
  const int64_t o0 = clamp_i64(a.offsets[e], 0, a.T), o1 = clamp_i64(a.offsets[e + 1], 0, a.T);
  const int64_t row0 = o0 + (int64_t)blockIdx.z * GEN_TOK;
  if (n >= a.N || row0 >= o1) return;
  const int rows = (int)(o1 - row0 < GEN_TOK ? o1 - row0 : GEN_TOK);

  float total[GEN_TOK];
#pragma unroll
  for (int r = 0; r < GEN_TOK; ++r) total[r] = 0.f;

  for (int term = 0; term < a.n_terms; ++term) {
    const uint8_t* wrow = a.packed[term] + (e * a.N + n) * a.Kp;
    const int64_t sbase = (e * a.N + n) * a.G;
    float y[GEN_TOK];
#pragma unroll
    for (int r = 0; r < GEN_TOK; ++r) y[r] = 0.f;
    for (int64_t g = 0; g < a.G; ++g) {
      const int64_t k0 = g * a.group;
      const int64_t k1 = k0 + a.group < a.K ? k0 + a.group : a.K;
      const float s = load_scale(a.w_scale[term], a.scale_dtype, sbase + g);
      if (INT8) {
        int acc[GEN_TOK];
#pragma unroll
        for (int r = 0; r < GEN_TOK; ++r) acc[r] = 0;
        for (int64_t k = k0 + lane; k < k1; k += 64) {
          const int t = decode_trit(wrow, k, a.fmt, lut);
#pragma unroll
          for (int r = 0; r < GEN_TOK; ++r)
            if (r < rows) acc[r] += t * (int)((const int8_t*)a.x)[(row0 + r) * a.K + k];
        }
#pragma unroll
        for (int r = 0; r < GEN_TOK; ++r) {
          const int sum = wave_sum(acc[r]);
          y[r] = __fadd_rn(y[r], __fmul_rn((float)sum, s));  // out += acc * w_scale[:, g]
        }
      } else {
        float acc[GEN_TOK];
#pragma unroll
        for (int r = 0; r < GEN_TOK; ++r) acc[r] = 0.f;
        for (int64_t k = k0 + lane; k < k1; k += 64) {
          const int t = decode_trit(wrow, k, a.fmt, lut);
          if (t != 0) {  // a zero trit never touches x, as in the reference's select-and-add loop
#pragma unroll
            for (int r = 0; r < GEN_TOK; ++r)
              if (r < rows) acc[r] += (float)t * load_act_f32(a.x, a.x_dtype, (row0 + r) * a.K + k);
          }
        }
#pragma unroll
        for (int r = 0; r < GEN_TOK; ++r) y[r] = __fadd_rn(y[r], __fmul_rn(wave_sum(acc[r]), s));
      }
    }
#pragma unroll
    for (int r = 0; r < GEN_TOK; ++r) {
      if (r < rows) {
        const float v = INT8 ? __fmul_rn(y[r], a.x_scale[row0 + r]) : y[r];
        total[r] = term == 0 ? v : __fadd_rn(total[r], v);
      }
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < GEN_TOK; ++r)
      if (r < rows) a.out[(row0 + r) * a.N + n] = __fadd_rn(a.out[(row0 + r) * a.N + n], total[r]);
  }
}

// ---- format kernels ------------------------------------------------------------------------

__global__ __launch_bounds__(256) void k_unpack(int8_t* __restrict__ trits, const uint8_t* __restrict__ packed,
                                                int64_t N, int64_t K, int64_t Kp, int fmt) {
  const int per = fmt == BP_TQ2 ? 4 : 5;
  const int64_t total = N * Kp;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t n = i / Kp, b = i % Kp;
    const unsigned v = packed[i];
    for (int d = 0; d < per; ++d) {
      const int64_t k = b * per + d;
      if (k < K) trits[n * K + k] = (int8_t)(fmt == BP_TQ2 ? (int)((v >> (2 * d)) & 3u) - 1 : tq1_trit(v, d));
    }
  }
}

__global__ __launch_bounds__(256) void k_pack(uint8_t* __restrict__ packed, const int8_t* __restrict__ trits,
                                              int64_t N, int64_t K, int64_t Kp, int fmt) {
  const int per = fmt == BP_TQ2 ? 4 : 5;
  const int64_t total = N * Kp;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t n = i / Kp, b = i % Kp;
    unsigned v = 0, w = 1;
    for (int d = 0; d < per; ++d) {
      const int64_t k = b * per + d;
      const unsigned u = k < K ? (unsigned)(((int)trits[n * K + k] + 1) & 0xff) : 1u;  // pad digit 1
      if (fmt == BP_TQ2) v |= u << (2 * d);
      else { v += u * w; w *= 3u; }
    }
    packed[i] = (uint8_t)v;
  }
}


// ---- pack / unpack with the trit side in 16-byte pieces (K a multiple of 16, 16-byte aligned trits): a workgroup takes
// SEG_BYTES packed bytes of one row, a thread four of them (16 or 20 trits); the trits cross LDS so that global memory
// sees them as consecutive 16-byte pieces whatever the 5-trit bytes' stride is. Same values as k_pack / k_unpack.
constexpr int SEG_BYTES = 1024;
template <int FMT>
__global__ __launch_bounds__(256) void k_unpack_seg(int8_t* __restrict__ trits, const uint8_t* __restrict__ packed, int64_t K, int64_t Kp) {
  constexpr int PER = FMT == BP_TQ2 ? 4 : 5;
  __shared__ __attribute__((aligned(16))) unsigned seg[256 * PER];
  const int64_t n = blockIdx.x, b0 = (int64_t)blockIdx.y * SEG_BYTES;
  const uint8_t* prow = packed + n * Kp + b0;
  const int64_t left = Kp - b0;  // packed bytes of the row from b0 on
  // TQ1: a byte's five trits from a table in LDS (entry v: trits 0..3 in one dword, trit 4 in the next), made by the
  // workgroup's 256 threads - five divisions per byte otherwise
  __shared__ unsigned digits[FMT == BP_TQ1 ? 512 : 1];
  if (FMT == BP_TQ1) {
    const unsigned v = threadIdx.x;
    digits[2 * v] = (unsigned)(tq1_trit(v, 0) & 0xff) | ((unsigned)(tq1_trit(v, 1) & 0xff) << 8) | ((unsigned)(tq1_trit(v, 2) & 0xff) << 16) |
                    ((unsigned)(tq1_trit(v, 3) & 0xff) << 24);
    digits[2 * v + 1] = (unsigned)(tq1_trit(v, 4) & 0xff);
    __syncthreads();
  }
  unsigned char tb[4 * PER];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int b = 4 * (int)threadIdx.x + j;
    const unsigned v = b < left ? prow[b] : 0u;
    if (FMT == BP_TQ1) {
      const unsigned lo = digits[2 * v], hi = digits[2 * v + 1];
      tb[PER * j] = (unsigned char)lo; tb[PER * j + 1] = (unsigned char)(lo >> 8); tb[PER * j + 2] = (unsigned char)(lo >> 16);
      tb[PER * j + 3] = (unsigned char)(lo >> 24); tb[PER * j + PER - 1] = (unsigned char)hi;
    } else {
#pragma unroll
      for (int d = 0; d < PER; ++d) tb[PER * j + d] = (unsigned char)((int)((v >> (2 * d)) & 3u) - 1);
    }
  }
#pragma unroll
  for (int i = 0; i < PER; ++i)
    seg[PER * threadIdx.x + i] = (unsigned)tb[4 * i] | ((unsigned)tb[4 * i + 1] << 8) | ((unsigned)tb[4 * i + 2] << 16) | ((unsigned)tb[4 * i + 3] << 24);
  __syncthreads();
  const int64_t k0 = b0 * PER;
  const int64_t count = K - k0 < (int64_t)SEG_BYTES * PER ? K - k0 : (int64_t)SEG_BYTES * PER;  // (a multiple of 16)
  uint4* dst = (uint4*)(trits + n * K + k0);
  for (int pc = threadIdx.x; pc < count / 16; pc += 256) dst[pc] = ((const uint4*)seg)[pc];
}

template <int FMT>
__global__ __launch_bounds__(256) void k_pack_seg(uint8_t* __restrict__ packed, const int8_t* __restrict__ trits, int64_t K, int64_t Kp) {
  constexpr int PER = FMT == BP_TQ2 ? 4 : 5;
  __shared__ __attribute__((aligned(16))) unsigned seg[256 * PER];
  const int64_t n = blockIdx.x, b0 = (int64_t)blockIdx.y * SEG_BYTES;
  const int64_t k0 = b0 * PER;
  const int64_t count = K - k0 < (int64_t)SEG_BYTES * PER ? K - k0 : (int64_t)SEG_BYTES * PER;
  const uint4* src = (const uint4*)(trits + n * K + k0);
  for (int pc = threadIdx.x; pc < SEG_BYTES * PER / 16; pc += 256)  // (past the row: trit 0, the pad digit 1)
    ((uint4*)seg)[pc] = pc < count / 16 ? src[pc] : make_uint4(0u, 0u, 0u, 0u);
  __syncthreads();
  unsigned char tb[4 * PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const unsigned w = seg[PER * threadIdx.x + i];
    tb[4 * i] = (unsigned char)w; tb[4 * i + 1] = (unsigned char)(w >> 8); tb[4 * i + 2] = (unsigned char)(w >> 16); tb[4 * i + 3] = (unsigned char)(w >> 24);
  }
  unsigned out = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    unsigned v = 0, mul = 1;
#pragma unroll
    for (int d = 0; d < PER; ++d) {
      const unsigned u = (unsigned)(((int)(signed char)tb[PER * j + d] + 1) & 0xff);
      if (FMT == BP_TQ2) v |= u << (2 * d);
      else { v += u * mul; mul *= 3u; }
    }
    out |= (v & 0xffu) << (8 * j);
  }
  const int64_t left = Kp - b0;
  const int b = 4 * (int)threadIdx.x;
  uint8_t* prow = packed + n * Kp + b0;
  if ((((uintptr_t)prow) & 3) == 0 && b + 3 < left) {
    *(unsigned*)(prow + b) = out;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (b + j < left) prow[b + j] = (uint8_t)(out >> (8 * j));
  }
}

__global__ __launch_bounds__(256) void k_expand(float* __restrict__ out, const void* __restrict__ in, int dtype, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = load_scale(in, dtype, i);
}

__global__ void k_lut(int8_t* lut) {
  for (int i = threadIdx.x; i < 256 * 5; i += blockDim.x) lut[i] = (int8_t)tq1_trit(i / 5, i % 5);
}

// One workgroup per activation row: absmax reduction, then the quantisation pass.
__global__ __launch_bounds__(256) void k_quant(int8_t* __restrict__ q, float* __restrict__ s, const void* __restrict__ x,
                                               int dtype, int64_t K) {
  __shared__ float part[4];
  const int64_t m = blockIdx.x;
  float amax = 0.f;
  bool nan = false;
  for (int64_t k = threadIdx.x; k < K; k += blockDim.x) {
    const float v = load_act_f32(x, dtype, m * K + k);
    nan |= v != v;
    amax = fmaxf(amax, fabsf(v));
  }
  if (nan) amax = __builtin_nanf("");
  float w = amax;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(w, off, 64);
    w = (w != w || o != o) ? __builtin_nanf("") : fmaxf(w, o);
  }
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = w;
  __syncthreads();
  float a = part[0];
  for (int i = 1; i < 4; ++i) a = (a != a || part[i] != part[i]) ? __builtin_nanf("") : fmaxf(a, part[i]);
  float sc = __fdiv_rn(a, 127.0f);
  sc = sc != sc ? sc : fmaxf(sc, 1e-8f);  // clamp(min=1e-8) keeps NaN
  if (threadIdx.x == 0) s[m] = sc;
  for (int64_t k = threadIdx.x; k < K; k += blockDim.x) {
    const float v = load_act_f32(x, dtype, m * K + k);
    float r = rintf(__fdiv_rn(v, sc));  // round half to even, like torch.round
    r = fminf(fmaxf(r, -127.f), 127.f);
    q[m * K + k] = (int8_t)(r != r ? 0 : (int)r);
  }
}

// The same for 16-bit activations in rows of whole 16-byte pieces (K % 8 == 0, K <= 8192, aligned pointers): a thread keeps
// its up to four pieces of the row in registers between the two passes, so the row is read once, in 16-byte loads, and
// written in 8-byte stores. Same arithmetic as k_quant, operation for operation.
constexpr int QUANT_VPT = 4;
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
template <int DT>
__global__ __launch_bounds__(256) void k_quant16(int8_t* __restrict__ q, float* __restrict__ s, const uint16_t* __restrict__ x, int64_t K) {
  __shared__ float part[4];
  const int64_t m = blockIdx.x;
  const int pieces = (int)(K / 8);
  u32x4 raw[QUANT_VPT];
  float amax = 0.f;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < QUANT_VPT; ++i) {
    const int pc = threadIdx.x + 256 * i;
    raw[i] = u32x4{0u, 0u, 0u, 0u};
    if (pc < pieces) raw[i] = *(const u32x4*)(x + m * K + 8 * (int64_t)pc);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint16_t h = (uint16_t)(raw[i][j >> 1] >> (16 * (j & 1)));
      const float v = DT == BP_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
      nan |= v != v;
      amax = fmaxf(amax, fabsf(v));
    }
  }
  if (nan) amax = __builtin_nanf("");
  float w = amax;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(w, off, 64);
    w = (w != w || o != o) ? __builtin_nanf("") : fmaxf(w, o);
  }
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = w;
  __syncthreads();
  float a = part[0];
  for (int i = 1; i < 4; ++i) a = (a != a || part[i] != part[i]) ? __builtin_nanf("") : fmaxf(a, part[i]);
  float sc = __fdiv_rn(a, 127.0f);
  sc = sc != sc ? sc : fmaxf(sc, 1e-8f);  // clamp(min=1e-8) keeps NaN
  if (threadIdx.x == 0) s[m] = sc;
#pragma unroll
  for (int i = 0; i < QUANT_VPT; ++i) {
    const int pc = threadIdx.x + 256 * i;
    unsigned out[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint16_t h = (uint16_t)(raw[i][j >> 1] >> (16 * (j & 1)));
      const float v = DT == BP_BF16 ? bf16_bits_to_f32(h) : f16_bits_to_f32(h);
      float r = rintf(__fdiv_rn(v, sc));  // round half to even, like torch.round
      r = fminf(fmaxf(r, -127.f), 127.f);
      out[j >> 2] |= ((unsigned)(r != r ? 0 : (int)r) & 0xffu) << (8 * (j & 3));
    }
    if (pc < pieces) *(u32x2*)(q + m * K + 8 * (int64_t)pc) = u32x2{out[0], out[1]};
  }
}

int grid_for(int64_t n) {
  int64_t g = (n + 255) / 256;
  return (int)(g < 1 ? 1 : (g > 65535 ? 65535 : g));
}

// BitNet b1.58 absmean quantizer fused with the packing (boilerplate/ternary/fit.py:78-96, boilerplate/qat/bitlinear.py:75-80):
// per row and group s = scale_dtype(sum |w| / count) - the sum taken in ascending k, the last group counting its own
// columns - then trit = s > 0 ? clamp(rint(w / max(s, 1e-30)), -1, 1) : 0, packed in the reference layout (pad digit 1).
// One workgroup per row: its G scales first (kept in LDS and written out), then its packed bytes.
constexpr int ABSMEAN_MAX_G = 8192;
__global__ __launch_bounds__(256) void k_absmean_pack(uint8_t* __restrict__ packed, void* __restrict__ scale, int8_t* __restrict__ trits,
                                                      const void* __restrict__ w, int w_dtype, int scale_dtype, int64_t K, int64_t Kp,
                                                      int64_t G, int64_t group, int fmt) {
  __shared__ float srow[ABSMEAN_MAX_G];
  const int64_t n = blockIdx.x;
  const int64_t wrow = n * K;
  for (int64_t g = threadIdx.x; g < G; g += blockDim.x) {
    const int64_t k0 = g * group, k1 = k0 + group < K ? k0 + group : K;
    float sum = 0.f;
    for (int64_t k = k0; k < k1; ++k) sum += fabsf(load_act_f32(w, w_dtype, wrow + k));
    const float mean = sum / (float)(k1 - k0);
    float rounded;
    if (scale_dtype == BP_F16) {
      const _Float16 h = (_Float16)mean;
      ((_Float16*)scale)[n * G + g] = h;
      rounded = (float)h;
    } else {
      const uint16_t b = f32_to_bf16_bits(mean);
      ((uint16_t*)scale)[n * G + g] = b;
      rounded = bf16_bits_to_f32(b);
    }
    srow[g] = rounded;
  }
  __syncthreads();
  const int per = fmt == BP_TQ2 ? 4 : 5;
  for (int64_t c = threadIdx.x; c < Kp; c += blockDim.x) {
    unsigned byte = 0, mul = 1;
    for (int i = 0; i < per; ++i) {
      const int64_t k = c * per + i;
      int t = 0;
      if (k < K) {
        const float s = srow[k / group];
        if (s > 0.f) {
          float r = rintf(load_act_f32(w, w_dtype, wrow + k) / fmaxf(s, 1e-30f));
          r = r < -1.f ? -1.f : r > 1.f ? 1.f : r;
          t = (int)r;  // (a NaN weight compares false twice and converts to 0)
        }
        if (trits) trits[wrow + k] = (int8_t)t;
      }
      const unsigned u = (unsigned)(t + 1);
      if (fmt == BP_TQ2) byte |= u << (2 * i);
      else { byte += u * mul; mul *= 3; }
    }
    packed[n * Kp + c] = (uint8_t)byte;
  }
}


// The same with the row staged in LDS as float32 (rows of whole 16-byte pieces at 16-byte aligned addresses that fit: the
// launcher's choice): the row is read once, in consecutive 16-byte pieces, where the kernel above reads it twice with
// a stride of one group between neighbouring threads in its first pass. Group g's values sit at g (group + 1) + i, so
// the threads that add up neighbouring groups - each in ascending k, the order of the kernel above: the same scales
// bit for bit - read different banks. LDS: K + G floats of the row, then the G rounded scales.
template <int WDT>
__global__ __launch_bounds__(256) void k_absmean_pack_lds(uint8_t* __restrict__ packed, void* __restrict__ scale, int8_t* __restrict__ trits,
                                                          const void* __restrict__ w, int scale_dtype, int64_t K, int64_t Kp,
                                                          int64_t G, int64_t group, int fmt) {
  extern __shared__ __attribute__((aligned(16))) float row[];
  constexpr int EPP = WDT == BP_F32 ? 4 : 8;  // elements per 16-byte piece
  float* srow = row + K + G;
  const int64_t n = blockIdx.x;
  const uint4* src = (const uint4*)((const char*)w + n * K * (WDT == BP_F32 ? 4 : 2));
  const int grp = (int)group, kk = (int)K;
  for (int pc = threadIdx.x; pc < kk / EPP; pc += 256) {
    const uint4 v = src[pc];
    float f[EPP];
    if (WDT == BP_F32) {
      f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
    } else {
      const unsigned q[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        f[2 * j % EPP] = WDT == BP_F16 ? f16_bits_to_f32((uint16_t)q[j]) : bf16_bits_to_f32((uint16_t)q[j]);
        f[(2 * j + 1) % EPP] = WDT == BP_F16 ? f16_bits_to_f32((uint16_t)(q[j] >> 16)) : bf16_bits_to_f32((uint16_t)(q[j] >> 16));
      }
    }
    const int k0 = EPP * pc;
    int g = k0 / grp, r = k0 - g * grp;
#pragma unroll
    for (int j = 0; j < EPP; ++j) {
      row[k0 + j + g] = f[j];
      if (++r == grp) { r = 0; ++g; }
    }
  }
  __syncthreads();
  for (int g = threadIdx.x; g < (int)G; g += 256) {
    const int k0 = g * grp, cnt = k0 + grp < kk ? grp : kk - k0;
    const float* p = row + k0 + g;
    float sum = 0.f;
    int i = 0;
    for (; i + 16 <= cnt; i += 16) {  // (sixteen reads on their way, then added in ascending k)
      float v[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) v[j] = p[i + j];
#pragma unroll
      for (int j = 0; j < 16; ++j) sum += fabsf(v[j]);
    }
    for (; i < cnt; ++i) sum += fabsf(p[i]);
    const float mean = sum / (float)cnt;
    float rounded;
    if (scale_dtype == BP_F16) {
      const _Float16 h = (_Float16)mean;
      ((_Float16*)scale)[n * G + g] = h;
      rounded = (float)h;
    } else {
      const uint16_t b = f32_to_bf16_bits(mean);
      ((uint16_t*)scale)[n * G + g] = b;
      rounded = bf16_bits_to_f32(b);
    }
    srow[g] = rounded;
  }
  __syncthreads();
  const int per = fmt == BP_TQ2 ? 4 : 5;
  for (int c = threadIdx.x; c < (int)Kp; c += 256) {
    unsigned byte = 0, mul = 1;
    const int kb = c * per;
    int g = kb / grp, r = kb - g * grp;
    for (int i = 0; i < per; ++i) {
      const int k = kb + i;
      int t = 0;
      if (k < kk) {
        // clamp(rint(w / max(s, 1e-30)), -1, 1) without the division: the rounded quotient exceeds 1/2 (and rounds to
        // +-1 or beyond) exactly when |w| / se > 1/2 + 2^-25, i.e. |w| - se / 2 > se 2^-25; the difference is exact
        // wherever the comparison is close (|w| within a factor of two of se / 2), the product always (se >= 1e-30).
        // A quotient of exactly 1/2 rounds to even, 0. NaN weights compare false: 0, as the conversion of a NaN gives.
        const float s = srow[g], w = row[k + g];
        const float se = fmaxf(s, 1e-30f);
        if (s > 0.f && fabsf(w) - 0.5f * se > se * 0x1p-25f) t = w < 0.f ? -1 : 1;
        if (trits) trits[n * K + k] = (int8_t)t;
        if (++r == grp) { r = 0; ++g; }
      }
      const unsigned u = (unsigned)(t + 1);
      if (fmt == BP_TQ2) byte |= u << (2 * i);
      else { byte += u * mul; mul *= 3; }
    }
    packed[n * Kp + c] = (uint8_t)byte;
  }
}

}  // namespace

int launch_general(const GemmArgs& a, hipStream_t s) {
  if (a.max_rows <= 0 || a.N == 0 || a.E == 0) return BP_OK;
  const int64_t zt = (a.max_rows + GEN_TOK - 1) / GEN_TOK;
  if (zt > 65535) return fail(BP_ERR_ARG, "too many rows per expert for one launch");
  const dim3 grid((unsigned)((a.N + GEN_WAVES - 1) / GEN_WAVES), (unsigned)a.E, (unsigned)zt);
  if (a.x_dtype == BP_I8) {
    note_kernel("general_i8");
    hipLaunchKernelGGL(k_general<true>, grid, dim3(GEN_WAVES * 64), 0, s, a);
  } else {
    note_kernel("general_float");
    hipLaunchKernelGGL(k_general<false>, grid, dim3(GEN_WAVES * 64), 0, s, a);
  }
  return check_launch("general ternary GEMM");
}

}  // namespace bp

using namespace bp;

static int fmt_dims(int fmt, int64_t N, int64_t K, int64_t* Kp) {
  if (fmt != BP_TQ1 && fmt != BP_TQ2) return fail(BP_ERR_ARG, "fmt must be 1 (TQ1) or 2 (TQ2)");
  if (K <= 0 || K > ((int64_t)1 << 40) || N < 0 || N > ((int64_t)1 << 40)) return fail(BP_ERR_ARG, "invalid N or K");
  const int64_t per = fmt == BP_TQ2 ? 4 : 5;
  *Kp = K / per + (K % per != 0);
  return BP_OK;
}

extern "C" int bp_unpack_trits(int8_t* trits, const uint8_t* packed, int64_t N, int64_t K, int fmt, void* stream) {
  int64_t Kp;
  if (int rc = fmt_dims(fmt, N, K, &Kp)) return rc;
  if (N == 0) return BP_OK;
  if (!trits || !packed) return fail(BP_ERR_ARG, "null pointer");
  if (K % 16 == 0 && ((uintptr_t)trits & 15) == 0 && N <= 0x7fffffff && (Kp + SEG_BYTES - 1) / SEG_BYTES <= 65535) {
    const dim3 grid((unsigned)N, (unsigned)((Kp + SEG_BYTES - 1) / SEG_BYTES));
    if (fmt == BP_TQ2) hipLaunchKernelGGL(k_unpack_seg<BP_TQ2>, grid, dim3(256), 0, (hipStream_t)stream, trits, packed, K, Kp);
    else hipLaunchKernelGGL(k_unpack_seg<BP_TQ1>, grid, dim3(256), 0, (hipStream_t)stream, trits, packed, K, Kp);
    return check_launch("unpack");
  }
  hipLaunchKernelGGL(k_unpack, dim3(grid_for(N * Kp)), dim3(256), 0, (hipStream_t)stream, trits, packed, N, K, Kp, fmt);
  return check_launch("unpack");
}

extern "C" int bp_pack_trits(uint8_t* packed, const int8_t* trits, int64_t N, int64_t K, int fmt, void* stream) {
  int64_t Kp;
  if (int rc = fmt_dims(fmt, N, K, &Kp)) return rc;
  if (N == 0) return BP_OK;
  if (!trits || !packed) return fail(BP_ERR_ARG, "null pointer");
  if (K % 16 == 0 && ((uintptr_t)trits & 15) == 0 && N <= 0x7fffffff && (Kp + SEG_BYTES - 1) / SEG_BYTES <= 65535) {
    const dim3 grid((unsigned)N, (unsigned)((Kp + SEG_BYTES - 1) / SEG_BYTES));
    if (fmt == BP_TQ2) hipLaunchKernelGGL(k_pack_seg<BP_TQ2>, grid, dim3(256), 0, (hipStream_t)stream, packed, trits, K, Kp);
    else hipLaunchKernelGGL(k_pack_seg<BP_TQ1>, grid, dim3(256), 0, (hipStream_t)stream, packed, trits, K, Kp);
    return check_launch("pack");
  }
  hipLaunchKernelGGL(k_pack, dim3(grid_for(N * Kp)), dim3(256), 0, (hipStream_t)stream, packed, trits, N, K, Kp, fmt);
  return check_launch("pack");
}

extern "C" int bp_expand_scales(float* out, const void* scale, int scale_dtype, int64_t n, void* stream) {
  if (scale_dtype != BP_F16 && scale_dtype != BP_BF16 && scale_dtype != BP_F32) return fail(BP_ERR_ARG, "scale dtype must be f16, bf16 or f32");
  if (n < 0) return fail(BP_ERR_ARG, "negative element count");
  if (n == 0) return BP_OK;
  if (!out || !scale) return fail(BP_ERR_ARG, "null pointer");
  hipLaunchKernelGGL(k_expand, dim3(grid_for(n)), dim3(256), 0, (hipStream_t)stream, out, scale, scale_dtype, n);
  return check_launch("expand_scales");
}

extern "C" int bp_tq1_lut(int8_t* lut, void* stream) {
  if (!lut) return fail(BP_ERR_ARG, "null pointer");
  hipLaunchKernelGGL(k_lut, dim3(1), dim3(256), 0, (hipStream_t)stream, lut);
  return check_launch("tq1_lut");
}

extern "C" int bp_quant_act_int8(int8_t* q, float* s, const void* x, int x_dtype, int64_t M, int64_t K, void* stream) {
  if (x_dtype != BP_BF16 && x_dtype != BP_F16 && x_dtype != BP_F32) return fail(BP_ERR_ARG, "activation dtype must be bf16, f16 or f32");
  if (M < 0 || K <= 0 || M > 0x7fffffff) return fail(BP_ERR_ARG, "invalid M or K");
  if (M == 0) return BP_OK;
  if (!q || !s || !x) return fail(BP_ERR_ARG, "null pointer");
  const bool pieces = x_dtype != BP_F32 && K % 8 == 0 && K <= 8 * 256 * QUANT_VPT && ((uintptr_t)x & 15) == 0 && ((uintptr_t)q & 7) == 0;
  if (pieces && x_dtype == BP_BF16) hipLaunchKernelGGL(k_quant16<BP_BF16>, dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, q, s, (const uint16_t*)x, K);
  else if (pieces) hipLaunchKernelGGL(k_quant16<BP_F16>, dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, q, s, (const uint16_t*)x, K);
  else hipLaunchKernelGGL(k_quant, dim3((unsigned)M), dim3(256), 0, (hipStream_t)stream, q, s, x, x_dtype, K);
  return check_launch("quant_act_int8");
}

extern "C" int bp_absmean_pack(uint8_t* packed, void* scale, int scale_dtype, int8_t* trits, const void* w, int w_dtype,
                               int64_t N, int64_t K, int64_t group, int fmt, void* stream) {
  int64_t Kp;
  if (int rc = fmt_dims(fmt, N, K, &Kp)) return rc;
  if (w_dtype != BP_BF16 && w_dtype != BP_F16 && w_dtype != BP_F32) return fail(BP_ERR_ARG, "weight dtype must be bf16, f16 or f32");
  if (scale_dtype != BP_F16 && scale_dtype != BP_BF16) return fail(BP_ERR_ARG, "scale_dtype must be float16 or bfloat16");
  if (group <= 0) return fail(BP_ERR_ARG, "weight must be a matrix with a nonempty input dimension and positive group");
  const int64_t G = K / group + (K % group != 0);
  if (G > ABSMEAN_MAX_G) return fail(BP_ERR_ARG, "more than %d scale groups per row", ABSMEAN_MAX_G);
  if (N > 0x7fffffff) return fail(BP_ERR_ARG, "too many rows");
  if (N == 0) return BP_OK;
  if (!packed || !scale || !w) return fail(BP_ERR_ARG, "null pointer");
  // rows of whole 16-byte pieces that fit LDS beside their scales: the kernel that reads its row once
  const int64_t epp = w_dtype == BP_F32 ? 4 : 8;
  const size_t lds = (size_t)(K + 2 * G) * 4;
  if (K % epp == 0 && ((uintptr_t)w & 15) == 0 && lds <= 128 * 1024 && K < ((int64_t)1 << 24)) {
    const dim3 grid((unsigned)N);
    const hipStream_t st = (hipStream_t)stream;
#define BP_ABSMEAN(DT)                                                                                                          \
  {                                                                                                                             \
    if (const int rc = raise_lds_limit<k_absmean_pack_lds<DT>>(128 * 1024)) return rc;                                          \
    hipLaunchKernelGGL(k_absmean_pack_lds<DT>, grid, dim3(256), lds, st, packed, scale, trits, w, scale_dtype, K, Kp, G, group, fmt); \
    return check_launch("absmean_pack");                                                                                       \
  }
    if (w_dtype == BP_F32) BP_ABSMEAN(BP_F32)
    if (w_dtype == BP_F16) BP_ABSMEAN(BP_F16)
    BP_ABSMEAN(BP_BF16)
#undef BP_ABSMEAN
  }
  hipLaunchKernelGGL(k_absmean_pack, dim3((unsigned)N), dim3(256), 0, (hipStream_t)stream, packed, scale, trits, w, w_dtype, scale_dtype, K, Kp,
                     G, group, fmt);
  return check_launch("absmean_pack");
}

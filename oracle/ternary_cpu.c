/* CPU oracle (plain C + OpenMP) for the ternary GEMM. TEST INFRASTRUCTURE ONLY.
 *
 * A restatement of the algorithm of the reference's CPU kernel
 * (boilerplate/kernels/csrc/boilerplate_cpu.cpp:19-128): for every output row the packed row is
 * expanded once into int8 trits, then for every activation row and every scale group the group sum
 * is formed with adds and subtracts only, multiplied by the group scale once, and the row total is
 * added into the caller's output (times the activation scale for int8 activations).
 *
 * Used by tests/ as a checker and by bench.py's cpu_baseline leg as the timed CPU port. The product
 * library never links or loads it. It is itself checked against the NumPy oracle
 * (oracle/ternary_oracle.py) and against the reference's own kernel built into oracle/_ref.
 *
 * Build: see oracle/Makefile (gcc -O3 -march=x86-64-v3 -fopenmp -shared).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#ifdef __AVX2__
#include <immintrin.h>
#endif

enum { BP_ORACLE_OK = 0, BP_ORACLE_BAD_DIMS = 1, BP_ORACLE_NOMEM = 2 };

int bp_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* boilerplate_cpu.cpp:19-32. TQ2: four 2-bit digits per byte, low bits first, trit = digit - 1.
 * TQ1: five base-3 digits per byte through the caller's 256 x 5 table. `dst` holds nb * per trits. */
static void expand_row(const uint8_t* src, int64_t K, int fmt, const int8_t* lut1, int8_t* dst) {
  if (fmt == 2) {
    const int64_t nb = (K + 3) / 4;
    for (int64_t b = 0; b < nb; ++b) {
      const unsigned v = src[b];
      dst[4 * b + 0] = (int8_t)((int)(v & 3u) - 1);
      dst[4 * b + 1] = (int8_t)((int)((v >> 2) & 3u) - 1);
      dst[4 * b + 2] = (int8_t)((int)((v >> 4) & 3u) - 1);
      dst[4 * b + 3] = (int8_t)((int)((v >> 6) & 3u) - 1);
    }
  } else {
    const int64_t nb = (K + 4) / 5;
    for (int64_t b = 0; b < nb; ++b) memcpy(dst + 5 * b, lut1 + 5 * (int64_t)src[b], 5);
  }
}

#ifdef __AVX2__
static inline int64_t hsum_i16(__m256i a16) {
  const __m256i lo = _mm256_cvtepi16_epi32(_mm256_castsi256_si128(a16));
  const __m256i hi = _mm256_cvtepi16_epi32(_mm256_extracti128_si256(a16, 1));
  const __m256i s = _mm256_add_epi32(lo, hi);
  __m128i q = _mm_add_epi32(_mm256_castsi256_si128(s), _mm256_extracti128_si256(s, 1));
  q = _mm_add_epi32(q, _mm_shuffle_epi32(q, 0x4E));
  q = _mm_add_epi32(q, _mm_shuffle_epi32(q, 0xB1));
  return (int64_t)_mm_cvtsi128_si32(q);
}
#endif

/* boilerplate_cpu.cpp:34-68: exact integer sum of +x, -x or 0 selected by the trit's sign. */
static int64_t signed_sum_i8(const int8_t* x, const int8_t* t, int64_t n) {
  int64_t i = 0, total = 0;
#ifdef __AVX2__
  __m256i a16 = _mm256_setzero_si256();
  int pending = 0;
  for (; i + 32 <= n; i += 32) {
    const __m256i xv = _mm256_loadu_si256((const __m256i*)(x + i));
    const __m256i tv = _mm256_loadu_si256((const __m256i*)(t + i));
    const __m256i s = _mm256_sign_epi8(xv, tv);
    a16 = _mm256_add_epi16(a16, _mm256_cvtepi8_epi16(_mm256_castsi256_si128(s)));
    a16 = _mm256_add_epi16(a16, _mm256_cvtepi8_epi16(_mm256_extracti128_si256(s, 1)));
    if (++pending == 64) { /* 64 * 2 * 127 < 32767: drain before an int16 lane can overflow */
      total += hsum_i16(a16);
      a16 = _mm256_setzero_si256();
      pending = 0;
    }
  }
  total += hsum_i16(a16);
#endif
  for (; i < n; ++i) total += (t[i] > 0 ? x[i] : 0) - (t[i] < 0 ? x[i] : 0);
  return total;
}

/* boilerplate_cpu.cpp:70-77: float activations, sum of the +1 entries minus sum of the -1 entries,
 * each accumulated sequentially in float32. */
static float signed_sum_f32(const float* x, const int8_t* t, int64_t n) {
  float plus = 0.f, minus = 0.f;
  for (int64_t i = 0; i < n; ++i) {
    plus += t[i] > 0 ? x[i] : 0.f;
    minus += t[i] < 0 ? x[i] : 0.f;
  }
  return plus - minus;
}

/* boilerplate_cpu.cpp:79-128. out [M, N] float32 is accumulated into (+=).
 * x: int8 [M, K] with x_scale [M] (x_is_i8 != 0) or float32 [M, K] (x_scale ignored).
 * packed [N, Kp] uint8, w_scale [N, G] float32, lut1 [256 * 5] int8. threads <= 0: OpenMP default. */
int bp_oracle_ternary_gemm(float* out, const void* x, int x_is_i8, const float* x_scale,
                           const uint8_t* packed, const float* w_scale, int64_t M, int64_t N, int64_t K,
                           int64_t group, int fmt, const int8_t* lut1, int threads) {
  if (K <= 0 || K > INT64_MAX / 128 || group <= 0 || (fmt != 1 && fmt != 2) || M < 0 || N < 0)
    return BP_ORACLE_BAD_DIMS;
  const int64_t per = fmt == 2 ? 4 : 5;
  const int64_t Kp = K / per + (K % per != 0);
  const int64_t G = K / group + (K % group != 0);
  const int64_t padded = Kp * per;
  const int8_t* x8 = x_is_i8 ? (const int8_t*)x : NULL;
  const float* xf = x_is_i8 ? NULL : (const float*)x;
  int failed = 0;
#ifdef _OPENMP
  const int nt = threads > 0 ? threads : omp_get_max_threads();
#pragma omp parallel num_threads(nt)
#endif
  {
    int8_t* trow = (int8_t*)malloc((size_t)padded + 64);
    if (!trow) {
#ifdef _OPENMP
#pragma omp atomic write
#endif
      failed = 1;
    }
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
    for (int64_t n = 0; n < N; ++n) {
      if (!trow) continue;
      expand_row(packed + n * Kp, K, fmt, lut1, trow);
      const float* s = w_scale + n * G;
      for (int64_t m = 0; m < M; ++m) {
        float y = 0.f;
        for (int64_t g = 0; g < G; ++g) {
          const int64_t k0 = g * group;
          const int64_t len = K - k0 < group ? K - k0 : group;
          const float a = x_is_i8 ? (float)signed_sum_i8(x8 + m * K + k0, trow + k0, len)
                                  : signed_sum_f32(xf + m * K + k0, trow + k0, len);
          y += s[g] * a;
        }
        out[m * N + n] += x_is_i8 ? y * x_scale[m] : y;
      }
    }
    free(trow);
  }
  (void)threads;
  return failed ? BP_ORACLE_NOMEM : BP_ORACLE_OK;
}

/* Row-by-row expansion of a packed matrix to int8 trits [N, K] (the reference's unpack,
 * boilerplate/ternary/pack.py:48-51,73-74, through the same per-row routine as the GEMM). */
int bp_oracle_unpack(int8_t* trits, const uint8_t* packed, int64_t N, int64_t K, int fmt, const int8_t* lut1) {
  if (K <= 0 || (fmt != 1 && fmt != 2) || N < 0) return BP_ORACLE_BAD_DIMS;
  const int64_t per = fmt == 2 ? 4 : 5;
  const int64_t Kp = K / per + (K % per != 0);
  int8_t* trow = (int8_t*)malloc((size_t)(Kp * per) + 64);
  if (!trow) return BP_ORACLE_NOMEM;
  for (int64_t n = 0; n < N; ++n) {
    expand_row(packed + n * Kp, K, fmt, lut1, trow);
    memcpy(trits + n * K, trow, (size_t)K);
  }
  free(trow);
  return BP_ORACLE_OK;
}

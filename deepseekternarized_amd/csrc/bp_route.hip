// Token-to-expert routing kernels around the grouped GEMM: stable counting sort of expert ids,
// row gather (the x[order // k] permute), and the two elementwise stages of an expert MLP
// (SwiGLU, weighted combine) with the reference engine's bf16 rounding points.
#include <mutex>

#include "bp_common.h"

// Histograms of bp_sort_by_expert_static: device memory that belongs to the library (one copy per GPU the library
// runs on, held until the process ends), so that entry point needs no workspace and allocates nothing. In host code
// the name `scratch` is only a stand-in: the array's device address is looked up once per device (g_scratch_ptr).
static __device__ __align__(256) int32_t scratch[16 * BP_SORT_STATIC_MAX_EXPERTS];  // 16 waves x E counters: 4 MiB

namespace bp {
namespace {

constexpr int64_t SORT_STATIC_MAX_E = BP_SORT_STATIC_MAX_EXPERTS;
constexpr int SORT_MAX_DEVICES = 64;
std::mutex g_scratch_mutex;
int32_t* g_scratch_ptr[SORT_MAX_DEVICES] = {};

constexpr int SORT_THREADS = 1024;
constexpr int SORT_WAVES = SORT_THREADS / 64;
static_assert(SORT_WAVES == 16, "the static histogram array is sized for 16 waves");
constexpr int64_t SORT_LDS_INTS = 32768;  // 128 KiB of per-wave histograms in LDS

// One workgroup. Wave w owns the contiguous segment [w*seg, (w+1)*seg) of ids.
// Pass 1: per-wave histograms. Scan: offsets and, per wave, the first output slot of each expert.
// Pass 2: every wave walks its segment in order, 64 ids at a time; lanes holding the same expert are
// ranked by lane index (ballot + popcount), so equal ids keep their input order (stable). `inv` (or NULL): the inverse
// permutation, inv[i] = the slot of id i in the order (ids outside [0, E) have none and keep what inv held).
__global__ __launch_bounds__(SORT_THREADS) void k_sort(int64_t* __restrict__ order, int64_t* __restrict__ offsets,
                                                        const int64_t* __restrict__ ids, int64_t n, int64_t E,
                                                        int32_t* __restrict__ ws, int32_t* __restrict__ bad, int64_t* __restrict__ inv) {
  extern __shared__ int32_t lds_hist[];
  int32_t* hist = ws ? ws : lds_hist;  // [SORT_WAVES][E]
  __shared__ int64_t carry;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int64_t i = threadIdx.x; i < SORT_WAVES * E; i += SORT_THREADS) hist[i] = 0;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  const int64_t seg = (n + SORT_WAVES - 1) / SORT_WAVES;
  const int64_t lo = wave * seg, hi = lo + seg < n ? lo + seg : n;
  int32_t* mine = hist + wave * E;
  for (int64_t i = lo + lane; i < hi; i += 64) {
    const int64_t id = ids[i];
    if (id >= 0 && id < E) atomicAdd(&mine[id], 1);
    else if (bad) *bad = 1;
  }
  if (ws) __threadfence();  // (histograms in device memory; in LDS the barrier orders them)
  __syncthreads();
  // exclusive scan over experts of the column sums; chunks of SORT_THREADS experts at a time: a scan inside every wave
  // (shuffles), then the waves' totals through LDS
  __shared__ int64_t wave_total[SORT_WAVES];
  for (int64_t e0 = 0; e0 < E; e0 += SORT_THREADS) {
    const int64_t e = e0 + threadIdx.x;
    int64_t cnt = 0;
    if (e < E)
      for (int w = 0; w < SORT_WAVES; ++w) cnt += hist[w * E + e];
    int64_t incl = cnt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int64_t up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int64_t chunk_total = 0;
    for (int w = 0; w < SORT_WAVES; ++w) {
      if (w < wave) incl += wave_total[w];
      chunk_total += wave_total[w];
    }
    const int64_t base = carry + incl - cnt;  // exclusive prefix for expert e
    if (e < E) {
      offsets[e] = base;
      int64_t run = base;
      for (int w = 0; w < SORT_WAVES; ++w) {  // turn counts into first slots per wave
        const int32_t c = hist[w * E + e];
        hist[w * E + e] = (int32_t)run;
        run += c;
      }
    }
    __syncthreads();  // (every thread has read carry and the waves' totals)
    if (threadIdx.x == 0) carry += chunk_total;
    __syncthreads();
  }
  if (threadIdx.x == 0) offsets[E] = carry;
  if (ws) __threadfence();  // (histograms in device memory; in LDS the barrier orders them)
  __syncthreads();
  // Pass 2, 64 ids at a time: every lane finds the lanes that hold its expert (one ballot per bit of the expert index),
  // the lowest of them claims the run of output slots with one atomic, and a lane's slot is the run's first plus the
  // number of lower lanes with the same expert.
  int nbits = 1;
  while (((int64_t)1 << nbits) < E) ++nbits;
  for (int64_t i0 = lo; i0 < hi; i0 += 64) {
    const int64_t i = i0 + lane;
    const bool live = i < hi;
    const int64_t id = live ? ids[i] : -1;
    const bool todo = live && id >= 0 && id < E;
    unsigned long long same = __ballot(todo);
    for (int bit = 0; bit < nbits; ++bit) {
      const unsigned long long set = __ballot(todo && ((id >> bit) & 1));
      same &= ((id >> bit) & 1) ? set : ~set;
    }
    if (todo) {  // (same holds this lane)
      const int leader = __ffsll((long long)same) - 1;
      int32_t first = 0;
      if (lane == leader) first = atomicAdd(&mine[id], (int32_t)__popcll(same));  // claims the run of slots
      first = __shfl(first, leader, 64);
      const int64_t slot = first + __popcll(same & ((1ull << lane) - 1ull));
      order[slot] = i;
      if (inv) inv[i] = slot;
    }
  }
}

// Few ids (n <= SORT_SMALL_N = 128): one pass, no histograms. Element i goes to slot #(valid ids below id_i) + #(equal ids
// before i) - the stable order - and offsets[e] = #(valid ids below e); every thread scans the ids held in LDS
// (a broadcast read per step). Decode batches sort a few dozen ids: this takes a quarter of the general kernel's time.
constexpr int SORT_SMALL_THREADS = 64;
constexpr int SORT_SMALL_N = 2 * SORT_SMALL_THREADS;  // (beyond ~150 ids the scan of all ids per element loses to the histograms)
__global__ __launch_bounds__(SORT_SMALL_THREADS) void k_sort_small(int64_t* __restrict__ order, int64_t* __restrict__ offsets,
                                                                    const int64_t* __restrict__ ids, int n, int64_t E,
                                                                    int32_t* __restrict__ bad) {
  __shared__ int32_t sid[SORT_SMALL_N];
  int32_t mine[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int i = threadIdx.x + q * SORT_SMALL_THREADS;
    mine[q] = 0x7fffffff;  // an id outside [0, E) is left out of the order, as in the general kernel
    if (i < n) {
      const int64_t id = ids[i];
      if (id >= 0 && id < E) mine[q] = (int32_t)id;
      else if (bad) *bad = 1;
    }
    sid[i] = mine[q];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int i = threadIdx.x + q * SORT_SMALL_THREADS;
    if (i < n && mine[q] != 0x7fffffff) {
      int rank = 0;
      for (int j = 0; j < n; ++j) {
        const int32_t v = sid[j];
        rank += (v < mine[q] || (v == mine[q] && j < i)) ? 1 : 0;
      }
      order[rank] = i;
    }
  }
  for (int64_t e = threadIdx.x; e <= E; e += SORT_SMALL_THREADS) {
    int cnt = 0;
    for (int j = 0; j < n; ++j) cnt += sid[j] < e ? 1 : 0;
    offsets[e] = cnt;
  }
}

__global__ __launch_bounds__(256) void k_gather(uint16_t* __restrict__ dst, const uint16_t* __restrict__ src,
                                                const int64_t* __restrict__ index, int64_t divisor, int64_t src_rows,
                                                int64_t row_halfs) {
  const int64_t r = blockIdx.x;
  int64_t srow = index[r] / divisor;
  srow = clamp_i64(srow, 0, src_rows - 1);
  const uint16_t* s = src + srow * row_halfs;
  uint16_t* d = dst + r * row_halfs;
  if ((row_halfs & 7) == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
    const uint4* s4 = (const uint4*)s;
    uint4* d4 = (uint4*)d;
    for (int64_t i = threadIdx.x; i < row_halfs / 8; i += blockDim.x) d4[i] = s4[i];
  } else {
    for (int64_t i = threadIdx.x; i < row_halfs; i += blockDim.x) d[i] = s[i];
  }
}

__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// h = bf16(bf16(silu(bf16 g)) * bf16 u)   (F.silu on a bf16 tensor computes in float32 and rounds once)
__global__ __launch_bounds__(256) void k_swiglu(uint16_t* __restrict__ h, const float* __restrict__ gate,
                                                const float* __restrict__ up, int64_t rows, int64_t I, int64_t ld) {
  const int64_t total = rows * I;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / I, c = i % I;
    const float g = round_bf16(gate[r * ld + c]);
    const float u = round_bf16(up[r * ld + c]);
    const float sg = round_bf16(g / (1.0f + expf(-g)));
    h[i] = f32_to_bf16_bits(sg * u);
  }
}

// The same, four columns per thread (16-byte loads, no division): I and ld multiples of 4, 16-byte aligned gate / up, 8-byte aligned h.
__global__ __launch_bounds__(256) void k_swiglu4(uint16_t* __restrict__ h, const float* __restrict__ gate,
                                                 const float* __restrict__ up, int64_t rows, int64_t I, int64_t ld) {
  const int64_t c = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (c >= I) return;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    const float4 g4 = *(const float4*)(gate + r * ld + c), u4 = *(const float4*)(up + r * ld + c);
    const float gs[4] = {g4.x, g4.y, g4.z, g4.w}, us[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float g = round_bf16(gs[i]);
      const float u = round_bf16(us[i]);
      const float sg = round_bf16(g / (1.0f + expf(-g)));
      o[i] = f32_to_bf16_bits(sg * u);
    }
    *(uint2*)(h + r * I + c) = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
  }
}

// out[t, :] = bf16-accumulated sum over the token's slots in ascending expert order.
// One workgroup per (token, 1024 columns): the slots' rows and weights are looked up once, in expert order, then
// every thread reads its 4 columns of all k rows (independent loads) and accumulates them in that order.
// Y16: the rows of y are bf16 already (the down projection rounded them itself: the rounding the sum starts with).
constexpr int COMBINE_COLS = 1024;
template <bool Y16>
__global__ __launch_bounds__(256) void k_combine(uint16_t* __restrict__ out, const float* __restrict__ y,
                                                 const int64_t* __restrict__ inv, const uint16_t* __restrict__ w,
                                                 const int64_t* __restrict__ experts, int64_t k, int64_t H) {
  const int64_t t = blockIdx.x;
  __shared__ int64_t expert_of[64];
  __shared__ int64_t row_of[64];
  __shared__ float weight_of[64];
  const int sl = threadIdx.x;
  int64_t my_expert = 0;
  if (sl < k) expert_of[sl] = my_expert = experts[t * k + sl];
  __syncthreads();
  if (sl < k) {  // position of slot sl in ascending expert order (ties: slot order), as a rank among the k slots
    int rank = 0;
    for (int j = 0; j < k; ++j) rank += (expert_of[j] < my_expert || (expert_of[j] == my_expert && j < sl)) ? 1 : 0;
    row_of[rank] = clamp_i64(inv[t * k + sl], 0, (int64_t)gridDim.x * k - 1);  // (a position outside y - from a caller's corrupt routing - reads a wrong row, not foreign memory)
    weight_of[rank] = bf16_bits_to_f32(w[t * k + sl]);
  }
  __syncthreads();
  const int64_t c0 = (int64_t)blockIdx.y * COMBINE_COLS + 4 * threadIdx.x;
  if (c0 >= H) return;
  if ((H & 3) == 0) {  // rows of y are 16-byte aligned: four columns per load
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < k; s0 += 8) {  // up to 8 rows in flight
      float4 v[8];
      const int ns = k - s0 < 8 ? (int)(k - s0) : 8;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        if (s < ns) {
          if (Y16) {
            const uint2 b = *(const uint2*)((const uint16_t*)y + row_of[s0 + s] * H + c0);
            v[s] = make_float4(__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u), __uint_as_float(b.y << 16), __uint_as_float(b.y & 0xffff0000u));
          } else {
            v[s] = *(const float4*)(y + row_of[s0 + s] * H + c0);
          }
        }
      }
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        if (s < ns) {
          const float ws = weight_of[s0 + s];
          const float e[4] = {v[s].x, v[s].y, v[s].z, v[s].w};
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] = round_bf16(acc[i] + round_bf16(round_bf16(e[i]) * ws));
        }
      }
    }
    const uint32_t lo = (uint32_t)f32_to_bf16_bits(acc[0]) | ((uint32_t)f32_to_bf16_bits(acc[1]) << 16);
    const uint32_t hi = (uint32_t)f32_to_bf16_bits(acc[2]) | ((uint32_t)f32_to_bf16_bits(acc[3]) << 16);
    *(uint2*)(out + t * H + c0) = make_uint2(lo, hi);
    return;
  }
  for (int64_t c = c0; c < H && c < c0 + 4; ++c) {
    float acc = 0.f;
    for (int s = 0; s < k; ++s) {
      const float v = Y16 ? bf16_bits_to_f32(((const uint16_t*)y)[row_of[s] * H + c]) : round_bf16(y[row_of[s] * H + c]);
      acc = round_bf16(acc + round_bf16(v * weight_of[s]));
    }
    out[t * H + c] = f32_to_bf16_bits(acc);
  }
}

// SwiGLU of the V4 engine's experts (boilerplate/engine/model.py:376-387): the two linears return bf16, everything after
// them is float32 - up clamped to [-limit, limit] and gate to at most limit when limit > 0, silu(gate) * up, times the
// routing weight of the row's (token, slot) pair - and the product is rounded to bf16 once, as w2's input.
// Row r of the expert-ordered tensors belongs to pair order[r]; weights f32 [pairs] (NULL: no weighting, a shared expert).
__global__ __launch_bounds__(256) void k_swiglu_v4(uint16_t* __restrict__ h, const float* __restrict__ gate, const float* __restrict__ up,
                                                    const float* __restrict__ weights, const int64_t* __restrict__ order, int64_t pairs,
                                                    float limit, int64_t rows, int64_t I, int64_t ld) {
  const int64_t c = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (c >= I) return;
  for (int64_t r = blockIdx.y; r < rows; r += gridDim.y) {
    float w = 1.0f;
    if (weights) w = weights[order ? clamp_i64(order[r], 0, pairs - 1) : r];
    float gs[4], us[4];
    if ((I & 3) == 0 && (ld & 3) == 0 && (((uintptr_t)gate | (uintptr_t)up) & 15) == 0) {
      const float4 g4 = *(const float4*)(gate + r * ld + c), u4 = *(const float4*)(up + r * ld + c);
      gs[0] = g4.x; gs[1] = g4.y; gs[2] = g4.z; gs[3] = g4.w;
      us[0] = u4.x; us[1] = u4.y; us[2] = u4.z; us[3] = u4.w;
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        gs[i] = c + i < I ? gate[r * ld + c + i] : 0.f;
        us[i] = c + i < I ? up[r * ld + c + i] : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float g = round_bf16(gs[i]), u = round_bf16(us[i]);
      if (limit > 0.f) {  // torch.clamp: a NaN stays a NaN
        u = u < -limit ? -limit : (u > limit ? limit : u);
        g = g > limit ? limit : g;
      }
      float v = (g / (1.0f + expf(-g))) * u;
      if (weights) v = w * v;
      if (c + i < I) h[r * I + c + i] = f32_to_bf16_bits(v);
    }
  }
}

// Combine of the V4 engine (boilerplate/engine/model.py:407-422): y = zeros float32; for each expert in ascending
// order y[token] += its bf16 output (already weighted before w2). out[t] = that float32 sum (OUT_BF16: cast once).
template <bool OUT_BF16, bool Y16>
__global__ __launch_bounds__(256) void k_combine_v4(void* __restrict__ out, const float* __restrict__ y, const int64_t* __restrict__ inv,
                                                     const int64_t* __restrict__ experts, int64_t k, int64_t H) {
  const int64_t t = blockIdx.x;
  __shared__ int64_t expert_of[64];
  __shared__ int64_t row_of[64];
  const int sl = threadIdx.x;
  int64_t my_expert = 0;
  if (sl < k) expert_of[sl] = my_expert = experts[t * k + sl];
  __syncthreads();
  if (sl < k) {
    int rank = 0;
    for (int j = 0; j < k; ++j) rank += (expert_of[j] < my_expert || (expert_of[j] == my_expert && j < sl)) ? 1 : 0;
    row_of[rank] = clamp_i64(inv[t * k + sl], 0, (int64_t)gridDim.x * k - 1);
  }
  __syncthreads();
  for (int64_t c = (int64_t)blockIdx.y * COMBINE_COLS + threadIdx.x; c < H && c < ((int64_t)blockIdx.y + 1) * COMBINE_COLS; c += 256) {
    float acc = 0.f;
    for (int s = 0; s < k; ++s) acc += Y16 ? bf16_bits_to_f32(((const uint16_t*)y)[row_of[s] * H + c]) : round_bf16(y[row_of[s] * H + c]);
    if (OUT_BF16) ((uint16_t*)out)[t * H + c] = f32_to_bf16_bits(acc);
    else ((float*)out)[t * H + c] = acc;
  }
}

// flag = 1 if an expert has more rows than `max_rows` (offsets clamped to [0, T] as the GEMM kernels clamp them)
__global__ __launch_bounds__(256) void k_check_rows(int32_t* __restrict__ flag, const int64_t* __restrict__ offsets, int64_t E, int64_t T,
                                                    int64_t max_rows) {
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < E; e += (int64_t)gridDim.x * 256) {
    const int64_t o0 = clamp_i64(offsets[e], 0, T), o1 = clamp_i64(offsets[e + 1], 0, T);
    if (o1 - o0 > max_rows) *flag = 1;
  }
}


// ---- the router's softmax and top-k (boilerplate/engine/standard.py:160-165): one wave per token, lane L holds the
// scores of experts L, L + 64, ... (up to ROUTE_PER_LANE of them). Softmax in float32 - the largest logit by a wave
// maximum, exp(x - max), the sum lane by lane in expert order and then across the wave in a fixed butterfly - then k
// rounds of a wave arg-max over (score, expert) with ties to the lower expert, the winner's entry taken out after each:
// the slots come out in descending score like torch.topk's. `renorm`: the k scores are divided by their sum
// (norm_topk_prob) before they are rounded to the output dtype.
constexpr int ROUTE_PER_LANE = 16;  // experts per lane at most: up to 1024 experts
template <int LDT, bool W_BF16, int PER /* experts per lane: E <= 64 PER */>
__global__ __launch_bounds__(256) void k_route_topk(void* __restrict__ weights, int64_t* __restrict__ experts, const void* __restrict__ logits,
                                                     int64_t T, int E, int k, int renorm) {
  const int lane = threadIdx.x & 63;
  const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;  // (uniform for the wave; no barrier below)
  float sc[PER];
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int e = lane + 64 * j;
    sc[j] = e < E ? load_act_f32(logits, LDT, t * E + e) : -INFINITY;
    mx = fmaxf(mx, sc[j]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    sc[j] = lane + 64 * j < E ? expf(sc[j] - mx) : 0.f;
    sum += sc[j];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
#pragma unroll
  for (int j = 0; j < PER; ++j) sc[j] = lane + 64 * j < E ? sc[j] / sum : -1.f;  // (scores are >= 0: -1 marks "no expert")
  float mine = 0.f;  // lane s keeps the score of slot s
  int mine_e = 0;
  float ksum = 0.f;
  for (int s = 0; s < k; ++s) {
    float best = -1.f;
    int best_e = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < PER; ++j)  // (ascending expert: a later equal score does not replace an earlier one)
      if (sc[j] > best) { best = sc[j]; best_e = lane + 64 * j; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off, 64);
      const int oe = __shfl_xor(best_e, off, 64);
      if (ov > best || (ov == best && oe < best_e)) { best = ov; best_e = oe; }
    }
    if ((best_e & 63) == lane) {  // the winner leaves its lane's list
#pragma unroll
      for (int j = 0; j < PER; ++j)
        if (j == (best_e >> 6)) sc[j] = -1.f;
    }
    if (lane == s) { mine = best; mine_e = best_e; }
    ksum += best;
  }
  if (lane < k) {
    const float v = renorm ? mine / ksum : mine;
    if (W_BF16) ((uint16_t*)weights)[t * k + lane] = f32_to_bf16_bits(v);
    else ((float*)weights)[t * k + lane] = v;
    experts[t * k + lane] = mine_e;
  }
}
}  // namespace
}  // namespace bp

using namespace bp;

extern "C" int64_t bp_sort_workspace_ints(int64_t n, int64_t E) {
  (void)n;
  if (E <= 0) return 0;
  return SORT_WAVES * E <= SORT_LDS_INTS ? 0 : SORT_WAVES * E;
}

static int launch_sort(int64_t* order, int64_t* offsets, const int64_t* ids, int64_t n, int64_t E, int32_t* hist_mem,
                       int32_t* bad, hipStream_t stream, int64_t* inv = nullptr) {
  if (!inv && n <= SORT_SMALL_N && E < ((int64_t)1 << 24)) {
    hipLaunchKernelGGL(k_sort_small, dim3(1), dim3(SORT_SMALL_THREADS), 0, stream, order, offsets, ids, (int)n, E, bad);
    return check_launch("sort_by_expert");
  }
  const size_t lds = hist_mem ? 0 : (size_t)(SORT_WAVES * (E > 0 ? E : 1)) * sizeof(int32_t);
  if (const int rc = raise_lds_limit<k_sort>((int)(SORT_LDS_INTS * 4))) return rc;
  hipLaunchKernelGGL(k_sort, dim3(1), dim3(SORT_THREADS), lds, stream, order, offsets, ids, n, E, hist_mem, bad, inv);
  return check_launch("sort_by_expert");
}

namespace bp {
// bp_sort_by_expert that also writes the inverse permutation (the MoE layer's preparation; arguments checked by its caller)
int sort_with_inverse(int64_t* order, int64_t* offsets, int64_t* inv, const int64_t* ids, int64_t n, int64_t E, int32_t* workspace,
                      int32_t* bad, hipStream_t stream) {
  return launch_sort(order, offsets, ids, n, E, bp_sort_workspace_ints(n, E) > 0 ? workspace : (int32_t*)nullptr, bad, stream, inv);
}
}  // namespace bp

extern "C" int bp_sort_by_expert(int64_t* order, int64_t* offsets, const int64_t* ids, int64_t n, int64_t E,
                                 int32_t* workspace, int32_t* bad, void* stream) {
  if (n < 0 || E < 0 || E > ((int64_t)1 << 24) || n > ((int64_t)1 << 31) - 1) return fail(BP_ERR_ARG, "invalid n or E");
  if (!offsets || (n > 0 && (!order || !ids))) return fail(BP_ERR_ARG, "null pointer");
  const int64_t need = bp_sort_workspace_ints(n, E);
  if (need > 0 && !workspace) return fail(BP_ERR_ARG, "sort_by_expert needs a workspace for this many experts");
  return launch_sort(order, offsets, ids, n, E, need > 0 ? workspace : (int32_t*)nullptr, bad, (hipStream_t)stream);
}

extern "C" int bp_sort_by_expert_static(int64_t* order, int64_t* offsets, const int64_t* ids, int64_t n, int64_t E,
                                        int32_t* bad, void* stream) {
  fail(BP_OK, "%s", "");  // (an earlier call's message does not outlive this one)
  if (n < 0 || E < 0 || n > ((int64_t)1 << 31) - 1) return fail(BP_ERR_ARG, "invalid n or E");
  if (E > SORT_STATIC_MAX_E)
    return fail(BP_ERR_ARG, "bp_sort_by_expert_static takes at most %lld experts (its histograms live in a fixed device array); "
                            "use bp_sort_by_expert with a workspace", (long long)SORT_STATIC_MAX_E);
  if (!offsets || (n > 0 && (!order || !ids))) return fail(BP_ERR_ARG, "null pointer");
  int32_t* hist_mem = nullptr;
  if (bp_sort_workspace_ints(n, E) > 0 && n > SORT_SMALL_N) {  // (otherwise the histograms fit in LDS, or none are used)
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= SORT_MAX_DEVICES) return fail(BP_ERR_LAUNCH, "cannot identify the current device");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {  // each GPU holds its own copy of the array at its own address
      void* p = nullptr;
      const hipError_t rc = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (rc != hipSuccess || !p) return fail(BP_ERR_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(rc));
      g_scratch_ptr[dev] = (int32_t*)p;
    }
    hist_mem = g_scratch_ptr[dev];
  }
  // the kernel zero-fills the SORT_WAVES * E counters it uses before counting: nothing of an earlier call is read
  return launch_sort(order, offsets, ids, n, E, hist_mem, bad, (hipStream_t)stream);
}

extern "C" int bp_gather_rows(void* dst, const void* src, const int64_t* index, int64_t divisor, int64_t rows,
                              int64_t src_rows, int64_t row_bytes, void* stream) {
  if (rows < 0 || src_rows < 0 || row_bytes <= 0 || (row_bytes & 1) || divisor <= 0 || rows > 0x7fffffff)
    return fail(BP_ERR_ARG, "invalid gather dimensions");
  if (rows == 0) return BP_OK;
  if (src_rows == 0) return fail(BP_ERR_ARG, "gather from an empty source");
  if (!dst || !src || !index) return fail(BP_ERR_ARG, "null pointer");
  hipLaunchKernelGGL(k_gather, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, (uint16_t*)dst,
                     (const uint16_t*)src, index, divisor, src_rows, row_bytes / 2);
  return check_launch("gather_rows");
}

extern "C" int bp_swiglu_bf16(void* h, const float* gate, const float* up, int64_t rows, int64_t I, int64_t ld_in, void* stream) {
  if (rows < 0 || I <= 0 || ld_in < I) return fail(BP_ERR_ARG, "invalid SwiGLU dimensions");
  if (rows == 0) return BP_OK;
  if (!h || !gate || !up) return fail(BP_ERR_ARG, "null pointer");
  if ((I & 3) == 0 && (ld_in & 3) == 0 && (((uintptr_t)gate | (uintptr_t)up) & 15) == 0 && ((uintptr_t)h & 7) == 0) {
    const dim3 grid((unsigned)((I + 1023) / 1024), (unsigned)(rows < 65535 ? rows : 65535));
    hipLaunchKernelGGL(k_swiglu4, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t*)h, gate, up, rows, I, ld_in);
    return check_launch("swiglu");
  }
  int64_t g = (rows * I + 255) / 256;
  if (g > 65535) g = 65535;
  hipLaunchKernelGGL(k_swiglu, dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, (uint16_t*)h, gate, up, rows, I, ld_in);
  return check_launch("swiglu");
}

namespace bp {
// the two combines with rows of y that are float32 (the entry points) or bf16 already (y16: bp_moe_layer_* after a down
// projection that wrote bf16)
int moe_combine(void* out, const void* y, bool y16, const int64_t* inv, const void* w, const int64_t* experts, int64_t T, int64_t k, int64_t H,
                void* stream) {
  if (T < 0 || k <= 0 || k > 64 || H <= 0 || T > 0x7fffffff) return fail(BP_ERR_ARG, "invalid combine dimensions (top-k up to 64)");
  if (T == 0) return BP_OK;
  if (!out || !y || !inv || !w || !experts) return fail(BP_ERR_ARG, "null pointer");
  const dim3 grid((unsigned)T, (unsigned)((H + COMBINE_COLS - 1) / COMBINE_COLS));
  if (y16) hipLaunchKernelGGL(k_combine<true>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t*)out, (const float*)y, inv, (const uint16_t*)w, experts, k, H);
  else hipLaunchKernelGGL(k_combine<false>, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t*)out, (const float*)y, inv, (const uint16_t*)w, experts, k, H);
  return check_launch("moe_combine");
}

int moe_combine_v4(void* out, int out_dtype, const void* y, bool y16, const int64_t* inv, const int64_t* experts, int64_t T, int64_t k, int64_t H,
                   void* stream) {
  if (T < 0 || k <= 0 || k > 64 || H <= 0 || T > 0x7fffffff) return fail(BP_ERR_ARG, "invalid combine dimensions (top-k up to 64)");
  if (out_dtype != BP_F32 && out_dtype != BP_BF16) return fail(BP_ERR_ARG, "the combined output is float32 or bf16");
  if (T == 0) return BP_OK;
  if (!out || !y || !inv || !experts) return fail(BP_ERR_ARG, "null pointer");
  const dim3 grid((unsigned)T, (unsigned)((H + COMBINE_COLS - 1) / COMBINE_COLS));
  const float* yf = (const float*)y;
  const hipStream_t s = (hipStream_t)stream;
  if (out_dtype == BP_BF16) {
    if (y16) hipLaunchKernelGGL((k_combine_v4<true, true>), grid, dim3(256), 0, s, out, yf, inv, experts, k, H);
    else hipLaunchKernelGGL((k_combine_v4<true, false>), grid, dim3(256), 0, s, out, yf, inv, experts, k, H);
  } else {
    if (y16) hipLaunchKernelGGL((k_combine_v4<false, true>), grid, dim3(256), 0, s, out, yf, inv, experts, k, H);
    else hipLaunchKernelGGL((k_combine_v4<false, false>), grid, dim3(256), 0, s, out, yf, inv, experts, k, H);
  }
  return check_launch("moe_combine_v4");
}
}  // namespace bp

extern "C" int bp_moe_combine_bf16(void* out, const float* y, const int64_t* inv, const void* w, const int64_t* experts,
                                   int64_t T, int64_t k, int64_t H, void* stream) {
  return bp::moe_combine(out, y, false, inv, w, experts, T, k, H, stream);
}

extern "C" int bp_swiglu_v4(void* h, const float* gate, const float* up, const float* weights, const int64_t* order, int64_t pairs,
                            float limit, int64_t rows, int64_t I, int64_t ld_in, void* stream) {
  if (rows < 0 || I <= 0 || ld_in < I || pairs < 0) return fail(BP_ERR_ARG, "invalid SwiGLU dimensions");
  if (rows == 0) return BP_OK;
  if (!h || !gate || !up) return fail(BP_ERR_ARG, "null pointer");
  if (weights && pairs == 0) return fail(BP_ERR_ARG, "routing weights without (token, slot) pairs");
  if (!(limit == limit)) return fail(BP_ERR_ARG, "swiglu_limit is NaN");
  const dim3 grid((unsigned)((I + 1023) / 1024), (unsigned)(rows < 65535 ? rows : 65535));
  hipLaunchKernelGGL(k_swiglu_v4, grid, dim3(256), 0, (hipStream_t)stream, (uint16_t*)h, gate, up, weights, order, pairs, limit, rows, I, ld_in);
  return check_launch("swiglu_v4");
}

extern "C" int bp_moe_combine_v4(void* out, int out_dtype, const float* y, const int64_t* inv, const int64_t* experts,
                                 int64_t T, int64_t k, int64_t H, void* stream) {
  return bp::moe_combine_v4(out, out_dtype, y, false, inv, experts, T, k, H, stream);
}

extern "C" int bp_route_topk(void* weights, int weights_dtype, int64_t* experts, const void* logits, int logits_dtype, int64_t T, int64_t E,
                             int64_t k, int renorm, void* stream) {
  if (T < 0 || E <= 0 || E > 64 * ROUTE_PER_LANE || k <= 0 || k > 64 || k > E) return fail(BP_ERR_ARG, "invalid routing dimensions (up to 1024 experts, top-k up to 64)");
  if (weights_dtype != BP_BF16 && weights_dtype != BP_F32) return fail(BP_ERR_ARG, "routing weights are bf16 or float32");
  if (logits_dtype != BP_BF16 && logits_dtype != BP_F16 && logits_dtype != BP_F32) return fail(BP_ERR_ARG, "router logits are bf16, fp16 or float32");
  if (T == 0) return BP_OK;
  if (!weights || !experts || !logits) return fail(BP_ERR_ARG, "null pointer");
  if ((T + 3) / 4 > 0x7fffffff) return fail(BP_ERR_ARG, "too many tokens");
  const dim3 grid((unsigned)((T + 3) / 4)), block(256);
  const hipStream_t s = (hipStream_t)stream;
#define BP_ROUTE_P(LDT, PER)                                                                                                                        \
  {                                                                                                                                                 \
    if (weights_dtype == BP_BF16) hipLaunchKernelGGL((k_route_topk<LDT, true, PER>), grid, block, 0, s, weights, experts, logits, T, (int)E, (int)k, renorm); \
    else hipLaunchKernelGGL((k_route_topk<LDT, false, PER>), grid, block, 0, s, weights, experts, logits, T, (int)E, (int)k, renorm);               \
  }
#define BP_ROUTE(LDT)                                 \
  if (logits_dtype == LDT) {                          \
    if (E <= 64) BP_ROUTE_P(LDT, 1)                   \
    else if (E <= 128) BP_ROUTE_P(LDT, 2)             \
    else if (E <= 256) BP_ROUTE_P(LDT, 4)             \
    else if (E <= 512) BP_ROUTE_P(LDT, 8)             \
    else BP_ROUTE_P(LDT, ROUTE_PER_LANE)              \
  }
  BP_ROUTE(BP_BF16) BP_ROUTE(BP_F16) BP_ROUTE(BP_F32)
#undef BP_ROUTE
#undef BP_ROUTE_P
  return check_launch("route_topk");
}

extern "C" int bp_check_max_rows(int32_t* flag, const int64_t* offsets, int64_t E, int64_t T, int64_t max_rows, void* stream) {
  if (E < 0 || T < 0 || max_rows < 0) return fail(BP_ERR_ARG, "invalid dimensions");
  if (E == 0) return BP_OK;
  if (!flag || !offsets) return fail(BP_ERR_ARG, "null pointer");
  int64_t g = (E + 255) / 256;
  if (g > 1024) g = 1024;
  hipLaunchKernelGGL(k_check_rows, dim3((unsigned)g), dim3(256), 0, (hipStream_t)stream, flag, offsets, E, T, max_rows);
  return check_launch("check_max_rows");
}

// One routed-expert MoE layer as one call: sort of the routing, row gather, gate|up grouped GEMM, SwiGLU, down grouped
// GEMM, weighted combine - the per-expert loop of boilerplate/engine/standard.py:156-176 after the router's top-k, with
// the same rounding points (every linear rounded to bf16, products with the routing weight rounded to bf16, the sum
// over a token's experts accumulated in bf16 in ascending expert order).
//
// Nothing is read back to the host. The reference sizes its grouped launch from `int(offsets.diff().max())`
// (boilerplate/kernels/ternary_cuda.py:97), a device-to-host copy in the middle of the layer; here a kernel writes
// the list of 32-row token tiles that exist (k_tile_list), and the grouped GEMMs run over that list. Up to 64 tokens
// no expert can have more than 64 rows, and the launch is sized by that bound instead (the small-batch kernels).
//
// All intermediate tensors live in a workspace the caller provides (bp_moe_layer_workspace_bytes): the library
// allocates nothing, so the call can be captured in a HIP graph.
#include <string.h>

#include "bp_mfma.h"

namespace bp {
int kernel_policy();  // bp_api.hip
int sort_with_inverse(int64_t* order, int64_t* offsets, int64_t* inv, const int64_t* ids, int64_t n, int64_t E, int32_t* workspace,
                      int32_t* bad, hipStream_t stream);  // bp_route.hip
int moe_combine(void* out, const void* y, bool y16, const int64_t* inv, const void* w, const int64_t* experts, int64_t T, int64_t k, int64_t H,
                void* stream);  // bp_route.hip
int moe_combine_v4(void* out, int out_dtype, const void* y, bool y16, const int64_t* inv, const int64_t* experts, int64_t T, int64_t k, int64_t H,
                   void* stream);
namespace {

constexpr int TILE_ROWS = 32;  // token tile of k_gemm_tq1 / k_gemm_tq2

// (expert, first row) of every 32-row token tile, in expert order; count[0] = their number. One workgroup; experts in
// chunks of 1024 with a running total.
__global__ __launch_bounds__(1024) void k_tile_list(int32_t* __restrict__ tiles, int32_t* __restrict__ count, const int64_t* __restrict__ offsets,
                                                    int64_t E, int64_t T, int64_t cap) {
  __shared__ int part[16];
  __shared__ int carry;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int64_t base = 0; base < E; base += 1024) {
    const int64_t e = base + threadIdx.x;
    int64_t o0 = 0, rows = 0;
    if (e < E) {
      o0 = clamp_i64(offsets[e], 0, T);
      const int64_t o1 = clamp_i64(offsets[e + 1], 0, T);
      rows = o1 > o0 ? o1 - o0 : 0;
    }
    const int mine = (int)((rows + TILE_ROWS - 1) / TILE_ROWS);
    int incl = mine;  // inclusive prefix sum within the wave
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (lane >= d) incl += up;
    }
    if (lane == 63) part[wave] = incl;
    __syncthreads();
    int before = carry;
    for (int w = 0; w < wave; ++w) before += part[w];
    int64_t at = before + incl - mine;
    for (int j = 0; j < mine; ++j, ++at) {
      if (at < cap) {
        tiles[2 * at] = (int32_t)e;
        tiles[2 * at + 1] = (int32_t)(o0 + (int64_t)j * TILE_ROWS);
      }
    }
    __syncthreads();
    if (threadIdx.x == 1023) carry = before + incl;
    __syncthreads();
  }
  if (threadIdx.x == 0) count[0] = carry < cap ? carry : (int)cap;
}

// The row gather xg[r] = x[order[r] / k] (rows of 16-byte pieces) and, in the same launch, the zero-fill of the two float32
// outputs that the GEMMs accumulate into (z0_16 = z1_16 = 0 where they write instead).
__global__ __launch_bounds__(256) void k_gather_zero(u32x4* __restrict__ xg, const u32x4* __restrict__ x, const int64_t* __restrict__ order, int64_t n,
                                                     int64_t k, int64_t T, int64_t row16, u32x4* __restrict__ z0, int64_t z0_16, u32x4* __restrict__ z1,
                                                     int64_t z1_16) {
  const int64_t gtid = (int64_t)blockIdx.x * 256 + threadIdx.x, gsz = (int64_t)gridDim.x * 256;
  for (int64_t w = gtid; w < n * row16; w += gsz) {
    const int64_t r = w / row16, c = w - r * row16;
    const int64_t src = clamp_i64(order[r] / k, 0, T - 1);
    xg[r * row16 + c] = x[src * row16 + c];
  }
  for (int64_t w = gtid; w < z0_16; w += gsz) z0[w] = u32x4{0u, 0u, 0u, 0u};
  for (int64_t w = gtid; w < z1_16; w += gsz) z1[w] = u32x4{0u, 0u, 0u, 0u};
}

__global__ __launch_bounds__(256) void k_zero16(u32x4* __restrict__ p, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256) p[i] = u32x4{0u, 0u, 0u, 0u};
}

// A few routed rows (n <= ROUTE_SMALL_N): the layer's whole preparation in one launch instead of five - stable sort of
// the expert ids (every workgroup ranks the ids for itself in LDS: element i goes to slot #(ids below id_i) + #(equal
// ids before i); workgroup 0 writes order, offsets and the inverse permutation), the row gather xg[r] = x[order[r] / k],
// and the zero-fill of the two float32 outputs that the small-batch kernels accumulate into - or, where the GEMMs run
// over the list of token tiles, that list (position r of the order starts a tile when it is a multiple of 32 rows into
// its expert; the tiles come out in expert order) instead of the zero-fill.
constexpr int ROUTE_SMALL_N = 256, ROUTE_SMALL_THREADS = 256;
__global__ __launch_bounds__(ROUTE_SMALL_THREADS) void k_route_small(int64_t* __restrict__ order, int64_t* __restrict__ offsets, int64_t* __restrict__ inv,
                                                                     const int64_t* __restrict__ ids, int n, int64_t E, int32_t* __restrict__ bad,
                                                                     u32x4* __restrict__ xg, const u32x4* __restrict__ x, int k, int64_t T, int64_t row16,
                                                                     u32x4* __restrict__ z0, int64_t z0_16, u32x4* __restrict__ z1, int64_t z1_16,
                                                                     int32_t* __restrict__ tiles, int32_t* __restrict__ tile_count, int64_t tile_cap) {
  __shared__ __attribute__((aligned(16))) int32_t sid[ROUTE_SMALL_N];  // (entries from n on: 0x7fffffff, "no expert")
  __shared__ int32_t ord[ROUTE_SMALL_N];
  __shared__ __attribute__((aligned(16))) int32_t tstart[ROUTE_SMALL_N];  // position r of the order starts a token tile
  const int i = threadIdx.x;
  int32_t mine = 0x7fffffff;  // an id outside [0, E) is left out of the order, as in bp_sort_by_expert
  if (i < n) {
    const int64_t id = ids[i];
    if (id >= 0 && id < E) mine = (int32_t)id;
    else if (bad && blockIdx.x == 0) *bad = 1;
  }
  sid[i] = mine;
  ord[i] = -1;
  tstart[i] = 0;
  __syncthreads();
  int rank = 0;
  if (i < n && mine != 0x7fffffff) {
    int lower = 0;  // rows of the experts before this one
    for (int j = 0; j < n; j += 4) {  // (four ids per LDS read; the padding compares as "after every expert")
      const int4 v = *(const int4*)&sid[j];
      lower += (v.x < mine ? 1 : 0) + (v.y < mine ? 1 : 0) + (v.z < mine ? 1 : 0) + (v.w < mine ? 1 : 0);
      rank += (v.x == mine && j < i ? 1 : 0) + (v.y == mine && j + 1 < i ? 1 : 0) + (v.z == mine && j + 2 < i ? 1 : 0) + (v.w == mine && j + 3 < i ? 1 : 0);
    }
    rank += lower;
    ord[rank] = i;
    if (((rank - lower) & (TILE_ROWS - 1)) == 0) tstart[rank] = 1;
    if (blockIdx.x == 0) {
      order[rank] = i;
      inv[i] = rank;
    }
  }
  if (blockIdx.x == 0) {
    for (int64_t e = i; e <= E; e += ROUTE_SMALL_THREADS) {
      int cnt = 0;
      for (int j = 0; j < n; j += 4) {
        const int4 v = *(const int4*)&sid[j];
        cnt += (v.x < e ? 1 : 0) + (v.y < e ? 1 : 0) + (v.z < e ? 1 : 0) + (v.w < e ? 1 : 0);
      }
      offsets[e] = cnt;
    }
  }
  __syncthreads();
  if (tiles && blockIdx.x == 0) {
    if (i < n && mine != 0x7fffffff && tstart[rank]) {
      int at = 0;  // tiles that start before this one
      for (int q = 0; q < rank; q += 4) {
        const int4 v = *(const int4*)&tstart[q];
        at += v.x + (q + 1 < rank ? v.y : 0) + (q + 2 < rank ? v.z : 0) + (q + 3 < rank ? v.w : 0);
      }
      if (at < tile_cap) {
        tiles[2 * at] = mine;
        tiles[2 * at + 1] = rank;
      }
    }
    if (i == ROUTE_SMALL_THREADS - 1) {
      int total = 0;
      for (int q = 0; q < n; q += 4) {  // (entries from n on are 0)
        const int4 v = *(const int4*)&tstart[q];
        total += v.x + v.y + v.z + v.w;
      }
      tile_count[0] = total < tile_cap ? total : (int)tile_cap;
    }
  }
  const int64_t gtid = (int64_t)blockIdx.x * ROUTE_SMALL_THREADS + i, gsz = (int64_t)gridDim.x * ROUTE_SMALL_THREADS;
  for (int64_t w = gtid; w < (int64_t)n * row16; w += gsz) {  // 16 bytes of a gathered row
    const int64_t r = w / row16, c = w - r * row16;
    const int o = ord[r];
    if (o >= 0) {
      int64_t src = o / k;
      src = src < T ? src : T - 1;
      xg[r * row16 + c] = x[src * row16 + c];
    }
  }
  for (int64_t w = gtid; w < z0_16; w += gsz) z0[w] = u32x4{0u, 0u, 0u, 0u};
  for (int64_t w = gtid; w < z1_16; w += gsz) z1[w] = u32x4{0u, 0u, 0u, 0u};
}

struct Carve {
  unsigned char* base;
  size_t used;
  void* take(size_t bytes) {
    void* p = base ? base + used : nullptr;
    used += (bytes + 255) & ~(size_t)255;
    return p;
  }
};

struct Plan {
  int64_t* order;
  int64_t* offsets;
  int64_t* inv;
  int32_t* sort_ws;
  int32_t* tiles;
  int32_t* tile_count;
  void* xg;       // gathered rows, bf16 [T k, H]
  int8_t* q;      // int8 activations of the wider of the two GEMM inputs
  float* q_scale;
  float* gu;      // f32 [T k, 2 I]
  void* h;        // bf16 [T k, I]
  float* y;       // f32 [T k, H]
  unsigned char* stage;  // converted activations of the GEMM in flight (bf16 activations)
  size_t stage_bytes;
  int64_t tile_cap;
  size_t bytes;
};

Plan plan(void* workspace, int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int act, int fmt) {
  Carve c = {(unsigned char*)workspace, 0};
  Plan p;
  const int64_t n = T * k;
  p.order = (int64_t*)c.take(8 * (size_t)n);
  p.offsets = (int64_t*)c.take(8 * (size_t)(E + 1));
  p.inv = (int64_t*)c.take(8 * (size_t)n);
  p.sort_ws = (int32_t*)c.take(4 * (size_t)bp_sort_workspace_ints(n, E));
  p.tile_cap = (n + TILE_ROWS - 1) / TILE_ROWS + E;
  p.tiles = (int32_t*)c.take(8 * (size_t)p.tile_cap);
  p.tile_count = (int32_t*)c.take(4);
  p.xg = c.take(2 * (size_t)n * H);
  p.q = (int8_t*)c.take(act == BP_I8 ? (size_t)n * (H > I ? H : I) : 0);
  p.q_scale = (float*)c.take(act == BP_I8 ? 4 * (size_t)n : 0);
  p.gu = (float*)c.take(4 * (size_t)n * 2 * I);
  p.h = c.take(2 * (size_t)n * I);
  p.y = (float*)c.take(4 * (size_t)n * H);
  p.stage_bytes = 0;
  if (act == BP_BF16) {
    const size_t a = gemm_tq2f_workspace_bytes(n, H, E), b = gemm_tq2f_workspace_bytes(n, I, E);
    p.stage_bytes = a > b ? a : b;
  }
  p.stage = (unsigned char*)c.take(p.stage_bytes);
  p.bytes = c.used;
  return p;
}

int zero(void* p, size_t bytes, hipStream_t s) {  // (a fill kernel, not a memset node: the call may be captured in a graph)
  const int64_t n16 = (int64_t)(bytes / 16);
  int64_t g = (n16 + 255) / 256;
  if (g > 8192) g = 8192;
  if (g > 0) hipLaunchKernelGGL(k_zero16, dim3((unsigned)g), dim3(256), 0, s, (u32x4*)p, n16);
  return check_launch("zero");
}

}  // namespace
}  // namespace bp

using namespace bp;

extern "C" size_t bp_moe_layer_workspace_bytes(int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int act, int fmt) {
  if (T < 0 || H <= 0 || I <= 0 || E <= 0 || k <= 0) return 0;
  return plan(nullptr, T, H, I, E, k, act, fmt).bytes;
}

// `v4`: the rounding points of the V4 engine (boilerplate/engine/model.py:376-387, 407-422) instead of the standard
// decoder's: float32 routing weights applied to the float32 SwiGLU product before the down projection, `limit` clamps,
// float32 accumulation over a token's experts, output float32 or cast once to bf16 (out_dtype).
static int moe_layer(bool v4, void* out, int out_dtype, float limit, const void* x, const int64_t* experts, const void* weights,
                     const uint8_t* const* gate_up_packed, const void* const* gate_up_scale,
                     const uint8_t* const* down_packed, const void* const* down_scale, int scale_dtype,
                     int n_terms, int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int64_t group, int fmt,
                     int act, void* workspace, size_t workspace_bytes, int32_t* bad, void* stream) {
  if (T < 0 || H <= 0 || I <= 0 || E <= 0 || E > 65535 || k <= 0 || k > 64 || k > E) return fail(BP_ERR_ARG, "invalid MoE layer dimensions (experts up to 65535, top-k up to 64)");
  if (T * k > ((int64_t)1 << 31) - 1 - 32 * E) return fail(BP_ERR_ARG, "too many routed rows for one call");
  if (fmt != BP_TQ1 && fmt != BP_TQ2) return fail(BP_ERR_ARG, "fmt must be 1 (TQ1) or 2 (TQ2)");
  if (act != BP_BF16 && act != BP_I8) return fail(BP_ERR_ARG, "act must be BP_BF16 or BP_I8");
  if (scale_dtype != BP_F32 && scale_dtype != BP_F16 && scale_dtype != BP_BF16) return fail(BP_ERR_ARG, "unexpected scale dtype");
  if (n_terms < 1 || n_terms > BP_MAX_TERMS) return fail(BP_ERR_ARG, "n_terms must be in 1..%d", BP_MAX_TERMS);
  if (group <= 0 || group > ((int64_t)1 << 24)) return fail(BP_ERR_ARG, "invalid group");
  if ((H % 8) != 0 || (I % 8) != 0) return fail(BP_ERR_ARG, "hidden and intermediate sizes must be multiples of 8 (16-byte rows)");
  if (T == 0) return BP_OK;
  if (!out || !x || !experts || !weights || !gate_up_packed || !gate_up_scale || !down_packed || !down_scale) return fail(BP_ERR_ARG, "null pointer");
  for (int t = 0; t < n_terms; ++t)
    if (!gate_up_packed[t] || !gate_up_scale[t] || !down_packed[t] || !down_scale[t]) return fail(BP_ERR_ARG, "null packed or scale pointer in term %d", t);
  const Plan p = plan(workspace, T, H, I, E, k, act, fmt);
  if (!workspace || workspace_bytes < p.bytes) return fail(BP_ERR_ARG, "the workspace must hold bp_moe_layer_workspace_bytes() = %zu bytes", p.bytes);
  if (((uintptr_t)workspace & 255) != 0) return fail(BP_ERR_ARG, "the workspace must be 256-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int64_t n = T * k;
  const int per = fmt == BP_TQ2 ? 4 : 5;

  int rc = BP_OK;
  // (the outputs' zero-fill rides along only where both GEMMs are going to accumulate: no tile list, and a policy that
  // lets them run; rows of 16-byte multiples: H % 8 == 0 is checked above)
  // Tokens beyond which the GEMMs run over the tile list. Up to 64 no expert can have more than 64 rows and the small-batch
  // kernels take the launch by that bound; TQ1 with bf16 activations changes over at 24 already: the launches of 8 rows
  // cost what their widest expert costs (an expert with 9 rows means a second pass over few CUs), the tile kernel a flat
  // 0.23 ms from 24 to 64 tokens on config 2's layer, where the small-batch kernels take 0.25 - 0.26 (and 0.18 - 0.21 below).
  const int64_t tiles_from = tuning().tiles >= 0 ? tuning().tiles : (fmt == BP_TQ1 && act == BP_BF16 ? 24 : 64);
  const bool tiles = T > tiles_from;
  const bool small = n <= ROUTE_SMALL_N && (((uintptr_t)x | (uintptr_t)p.xg) & 15) == 0;
  const bool aligned16 = (((uintptr_t)x | (uintptr_t)p.xg) & 15) == 0;
  const bool prezeroed = aligned16 && !tiles;  // the zero-fill rides along with the gather (the GEMMs over the tile list write instead of accumulate)
  // The gate | up projection as the grouped GEMM over converted activations with SwiGLU in its epilogue (bf16 h written,
  // no float32 gate | up rows), where that kernel takes the call: over the tile list, bf16 activations. Its conversion
  // pass then also does the row gather (rows read through `order`): no routed copy of the activations is written.
  GemmArgs fused;
  memset(&fused, 0, sizeof(fused));
  bool fuse = false;
  if (tiles && act == BP_BF16 && p.stage_bytes && kernel_policy() != 1 && tuning().glu != 'n' && tuning().tq2g != 'b') {
    GemmArgs& a = fused;
    a.out = p.gu; a.x = p.xg; a.offsets = p.offsets; a.x_dtype = act;
    for (int t = 0; t < n_terms; ++t) { a.packed[t] = gate_up_packed[t]; a.w_scale[t] = gate_up_scale[t]; }
    a.scale_dtype = scale_dtype; a.n_terms = n_terms; a.fmt = fmt;
    a.T = n; a.N = 2 * I; a.K = H; a.Kp = (H + per - 1) / per; a.G = (H + group - 1) / group; a.group = group; a.E = E;
    a.stage = p.stage; a.stage_bytes = (int64_t)p.stage_bytes;
    a.tiles = p.tiles; a.tile_count = p.tile_count; a.tile_cap = p.tile_cap;
    a.overwrite = 1; a.max_rows = TILE_ROWS;
    a.glu_h = (uint16_t*)p.h; a.glu_v4 = v4 ? 1 : 0; a.glu_limit = limit;
    a.glu_weights = v4 ? (const float*)weights : nullptr; a.glu_order = p.order; a.glu_pairs = n;
    if (aligned16 && tuning().glu != 'g') {  // (development: BP_TUNE_GLU=g keeps the gather a launch of its own)
      a.x = x; a.x_index = p.order; a.x_div = k; a.x_rows = T;
    }
    fuse = gemm_tiles_supported(a) && gemm_tq2f_applies(a) == BP_OK;
  }
  if (small) {
    const int64_t z0 = prezeroed ? (int64_t)(4 * (size_t)n * 2 * I / 16) : 0, z1 = prezeroed ? (int64_t)(4 * (size_t)n * H / 16) : 0;
    const int64_t row16 = fuse && fused.x_index ? 0 : H / 8;  // (no rows to copy where the gate | up launch reads them through `order`)
    int64_t g = (z0 + z1 + (int64_t)n * row16 + ROUTE_SMALL_THREADS - 1) / ROUTE_SMALL_THREADS;
    g = g < 1 ? 1 : (g > 256 ? 256 : g);
    hipLaunchKernelGGL(k_route_small, dim3((unsigned)g), dim3(ROUTE_SMALL_THREADS), 0, s, p.order, p.offsets, p.inv, experts, (int)n, E, bad,
                       (u32x4*)p.xg, (const u32x4*)x, (int)k, T, row16, (u32x4*)p.gu, z0, (u32x4*)p.y, z1, tiles ? p.tiles : nullptr, p.tile_count,
                       p.tile_cap);
    if ((rc = check_launch("route_small")) != BP_OK) return rc;
  } else {
    if ((rc = sort_with_inverse(p.order, p.offsets, p.inv, experts, n, E, p.sort_ws, bad, s)) != BP_OK) return rc;
    if (fuse && fused.x_index) {
      // (no routed copy of the activations: the gate | up launch's conversion pass reads them through `order`)
    } else if (aligned16) {
      const int64_t z0 = prezeroed ? (int64_t)(4 * (size_t)n * 2 * I / 16) : 0, z1 = prezeroed ? (int64_t)(4 * (size_t)n * H / 16) : 0;
      int64_t g = (z0 + z1 + n * (H / 8) + 255) / 256;
      g = g < 1 ? 1 : (g > 4096 ? 4096 : g);
      hipLaunchKernelGGL(k_gather_zero, dim3((unsigned)g), dim3(256), 0, s, (u32x4*)p.xg, (const u32x4*)x, p.order, n, k, T, H / 8, (u32x4*)p.gu, z0,
                         (u32x4*)p.y, z1);
      if ((rc = check_launch("gather_zero")) != BP_OK) return rc;
    } else if ((rc = bp_gather_rows(p.xg, x, p.order, k, n, T, 2 * H, s)) != BP_OK) return rc;
  }

  // `o16`: the caller takes bf16 rows (the combine rounds the down projection's rows to bf16 first); set to whether
  // the launch wrote them - the grouped GEMM over converted activations does, into the same buffer.
  auto gemm = [&](float* o, const void* in, const uint8_t* const* packed, const void* const* scale, int64_t N, int64_t K, bool tiles, bool* o16) -> int {
    const bool want16 = o16 && *o16;
    if (o16) *o16 = false;
    GemmArgs a;
    memset(&a, 0, sizeof(a));
    a.out = o;
    a.x = in;
    a.offsets = p.offsets;
    a.x_dtype = act;
    if (act == BP_I8) {
      if (const int q = bp_quant_act_int8(p.q, p.q_scale, in, BP_BF16, n, K, s)) return q;
      a.x = p.q;
      a.x_scale = p.q_scale;
    }
    for (int t = 0; t < n_terms; ++t) { a.packed[t] = packed[t]; a.w_scale[t] = scale[t]; }
    a.scale_dtype = scale_dtype; a.n_terms = n_terms; a.fmt = fmt;
    a.T = n; a.N = N; a.K = K; a.Kp = (K + per - 1) / per; a.G = (K + group - 1) / group; a.group = group; a.E = E;
    a.max_rows = T < n ? T : n;  // an expert has at most one row per token
    if (p.stage_bytes) {
      a.stage = p.stage;
      a.stage_bytes = (int64_t)p.stage_bytes;
    }
    if (tiles) {
      a.tiles = p.tiles; a.tile_count = p.tile_count; a.tile_cap = p.tile_cap;
      if (kernel_policy() != 1 && gemm_tiles_supported(a)) {
        a.overwrite = 1;
        a.max_rows = TILE_ROWS;
        if (want16 && tuning().glu != 'n' && tuning().tq2g != 'b') {
          a.out16 = (uint16_t*)o;
          if (gemm_tq2f_applies(a) == BP_OK) {
            *o16 = true;
            return launch_gemm_tq2f(a, s);
          }
          a.out16 = nullptr;
        }
        return run_gemm(a, s);
      }
      a.tiles = nullptr;  // no tile kernel for this shape: the launch covers the bound (every expert up to T rows)
    }
    if (!prezeroed)
      if (const int z = zero(o, 4 * (size_t)n * N, s)) return z;
    return run_gemm(a, s);
  };
  if (tiles && !small) {
    hipLaunchKernelGGL(k_tile_list, dim3(1), dim3(1024), 0, s, p.tiles, p.tile_count, p.offsets, E, n, p.tile_cap);
    if ((rc = check_launch("tile_list")) != BP_OK) return rc;
  }
  if (fuse) {
    rc = launch_gemm_tq2f(fused, s);
  } else {
    if ((rc = gemm(p.gu, p.xg, gate_up_packed, gate_up_scale, 2 * I, H, tiles, nullptr)) != BP_OK) return rc;
    if (v4) rc = bp_swiglu_v4(p.h, p.gu, p.gu + I, (const float*)weights, p.order, n, limit, n, I, 2 * I, s);
    else rc = bp_swiglu_bf16(p.h, p.gu, p.gu + I, n, I, 2 * I, s);
  }
  if (rc != BP_OK) return rc;
  bool y16 = true;
  if ((rc = gemm(p.y, p.h, down_packed, down_scale, H, I, tiles, &y16)) != BP_OK) return rc;
  if (fuse) note_kernel_suffix(fused.x_index ? "+glu+gather" : "+glu");  // (bp_last_kernel: the down projection's kernel, and that the gate | up one applied SwiGLU)
  if (y16) note_kernel_suffix("+y16");  // (... and that the down projection wrote bf16 rows)
  if (v4) return moe_combine_v4(out, out_dtype, p.y, y16, p.inv, experts, T, k, H, s);
  return moe_combine(out, p.y, y16, p.inv, weights, experts, T, k, H, s);
}

extern "C" int bp_moe_layer_bf16(void* out, const void* x, const int64_t* experts, const void* weights,
                                 const uint8_t* const* gate_up_packed, const void* const* gate_up_scale,
                                 const uint8_t* const* down_packed, const void* const* down_scale, int scale_dtype,
                                 int n_terms, int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int64_t group, int fmt,
                                 int act, void* workspace, size_t workspace_bytes, int32_t* bad, void* stream) {
  return moe_layer(false, out, BP_BF16, 0.f, x, experts, weights, gate_up_packed, gate_up_scale, down_packed, down_scale, scale_dtype,
                   n_terms, T, H, I, E, k, group, fmt, act, workspace, workspace_bytes, bad, stream);
}

extern "C" int bp_moe_layer_v4(void* out, int out_dtype, const void* x, const int64_t* experts, const float* weights, float swiglu_limit,
                               const uint8_t* const* gate_up_packed, const void* const* gate_up_scale,
                               const uint8_t* const* down_packed, const void* const* down_scale, int scale_dtype,
                               int n_terms, int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int64_t group, int fmt,
                               int act, void* workspace, size_t workspace_bytes, int32_t* bad, void* stream) {
  if (out_dtype != BP_F32 && out_dtype != BP_BF16) return fail(BP_ERR_ARG, "the layer's output is float32 or bf16");
  if (!(swiglu_limit == swiglu_limit) || swiglu_limit < 0.f) return fail(BP_ERR_ARG, "swiglu_limit must be 0 (no clamp) or positive");
  return moe_layer(true, out, out_dtype, swiglu_limit, x, experts, weights, gate_up_packed, gate_up_scale, down_packed, down_scale, scale_dtype,
                   n_terms, T, H, I, E, k, group, fmt, act, workspace, workspace_bytes, bad, stream);
}

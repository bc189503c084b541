// Shared declarations for the gfx950 ternary kernels: error reporting, dtype helpers, launch
// argument blocks. Host and device code of libbp_ternary_hip.so include this.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../include/bp_ternary.h"

namespace bp {

// ---- host-side error plumbing (thread local, surfaced through bp_last_error) ----
int fail(int code, const char* fmt, ...);
void note_kernel(const char* name);
void note_kernel_suffix(const char* suffix);  // ... appended to the name noted last
int check_launch(const char* what);

// ---- argument block of one grouped GEMM call (validated by the C entry point) ----
struct GemmArgs {
  float* out;
  const void* x;
  const float* x_scale;
  const int64_t* offsets;
  const uint8_t* packed[BP_MAX_TERMS];
  const void* w_scale[BP_MAX_TERMS];
  int x_dtype, scale_dtype, n_terms, fmt;
  int64_t T, N, K, Kp, G, group, E, max_rows;
  // Tile-list mode of the 32-token-tile kernels (set by callers that keep the routing on the device, where the widest
  // expert's row count is unknown to the host): tiles = (expert, first row) pairs of the token tiles that exist, in
  // expert order, tile_count[0] of them (device memory, written by a kernel earlier on the stream); the launch covers
  // tile_cap entries and workgroups past the count leave at once. NULL: token tiles are counted by blockIdx.z up to max_rows.
  const int32_t* tiles;
  const int32_t* tile_count;
  int64_t tile_cap;
  int overwrite;  // tile-list mode: the kernel's result replaces `out` instead of being added to it (one launch covers all of K and all terms)
  // Workspace of the caller for kernels that convert the activations in a pass of their own (NULL: those kernels are not used).
  unsigned char* stage;
  int64_t stage_bytes;
  // SwiGLU in the epilogue of the grouped GEMM over converted activations (glu_h != NULL; tile-list mode with overwrite):
  // the N output rows are N / 2 gate rows followed by N / 2 up rows, and the kernel writes bf16 glu_h[T, N / 2] instead
  // of `out`, with the rounding points of bp_swiglu_bf16 (glu_v4 = 0) or of bp_swiglu_v4 (glu_v4 = 1: clamp by glu_limit
  // when positive, float32 product times glu_weights[glu_order[row]] when glu_weights is set, one rounding to bf16).
  // Row gather in the conversion pass of that kernel (x_index != NULL): row r of the launch is row
  // x_index[r] / x_div of x, which has x_rows rows (the routed copy of the activations is never materialised).
  const int64_t* x_index;
  int64_t x_div, x_rows;
  uint16_t* out16;  // (the same kernel, tile-list mode with overwrite) bf16 out16[T, N] is written instead of float32 `out`
  uint16_t* glu_h;
  int glu_v4;
  float glu_limit;
  const float* glu_weights;
  const int64_t* glu_order;
  int64_t glu_pairs;
};

__device__ __forceinline__ int64_t clamp_i64(int64_t v, int64_t lo, int64_t hi) { return v < lo ? lo : (v > hi ? hi : v); }

// Which token tile of 32 rows a workgroup takes: `slot` is its expert (list entry in tile-list mode), z its token tile.
struct TileRef {
  int64_t e, tok0, o1;
  bool live;
};
__device__ __forceinline__ TileRef tile_ref(const GemmArgs& a, int64_t slot, unsigned z) {
  TileRef r = {0, 0, 0, false};
  if (a.tiles) {
    if (slot >= a.tile_count[0] || slot >= a.tile_cap) return r;
    r.e = a.tiles[2 * slot];
    r.tok0 = a.tiles[2 * slot + 1];
    r.o1 = clamp_i64(a.offsets[r.e + 1], 0, a.T);
  } else {
    if (slot >= a.E) return r;
    r.e = slot;
    r.o1 = clamp_i64(a.offsets[slot + 1], 0, a.T);
    r.tok0 = clamp_i64(a.offsets[slot], 0, a.T) + (int64_t)z * 32;
  }
  r.live = r.tok0 < r.o1;
  return r;
}

// Which token tile and which block of output rows a workgroup of a 32-token-tile kernel takes, from its linear index.
// Workgroups are dealt to the 8 XCDs round-robin by linear index and each XCD has its own L2. The row blocks of a token
// tile read the same activations and the token tiles of an expert the same weights, so an XCD takes its experts one after
// the other, an expert's token tiles one after the other and a tile's row blocks one after the other: the workgroups
// that run on it at one time share what they stream through its L2. In tile-list mode an expert's tiles are neighbours
// in the list, and an XCD takes the list in runs of TILE_RUN entries.
constexpr int TILE_RUN = 4;
__device__ __forceinline__ TileRef tile_of_workgroup(const GemmArgs& a, unsigned linear, int row_blocks, int& row_block) {
  const unsigned xcd = linear & 7;
  unsigned q = linear >> 3;
  row_block = (int)(q % (unsigned)row_blocks);
  q /= (unsigned)row_blocks;
  if (a.tiles) return tile_ref(a, (int64_t)(q / TILE_RUN) * (8 * TILE_RUN) + xcd * TILE_RUN + q % TILE_RUN, 0);
  const unsigned tiles_per_expert = (unsigned)((a.max_rows + 31) / 32);
  return tile_ref(a, xcd + 8 * (int64_t)(q / tiles_per_expert), q % tiles_per_expert);
}
// Workgroups of such a launch (-1: more than a grid's x extent holds).
inline int64_t tile_workgroups(const GemmArgs& a, int64_t row_blocks) {
  const int64_t slots = a.tiles ? a.tile_cap : a.E, per_round = a.tiles ? 8 * TILE_RUN : 8;
  const int64_t z = a.tiles ? 1 : (a.max_rows + 31) / 32;
  const int64_t rounds = (slots + per_round - 1) / per_round;
  if (z > 0x7fffffff / (row_blocks * per_round) || rounds > 0x7fffffff / (row_blocks * per_round * z)) return -1;
  return row_blocks * per_round * rounds * z;
}

// Development overrides of the kernel selection (environment variables BP_TUNE_*), read once when the library is first
// used; bp_reload_tuning() reads them again (the tests switch kernels that way). 0 / unset = automatic.
struct Tuning {
  int r;       // BP_TUNE_R: 16-row tiles per wave of the TQ2 kernel (1, 2)
  int waves;   // BP_TUNE_WAVES: waves per workgroup (8, 16)
  char tq1;    // BP_TUNE_TQ1: 'l' table-lookup GEMV, 'm' 16-token MFMA kernel, 'c' the chunk-per-wave GEMV wherever it can run, 'r' never (first letter of the value)
  char tq2g;   // BP_TUNE_TQ2G: 'b' (bf16) never the fp8 x fp4 grouped GEMM over converted activations, 'f' (fp4) wherever it can run
  char tq2v;   // BP_TUNE_TQ2V: 'k' the K-split fp8 x fp4 TQ2 GEMV wherever it can run, 'n' never
  int f4w;     // BP_TUNE_F4W: waves per workgroup of the fp8 x fp4 GEMV (8, 16)
  int f4t;     // BP_TUNE_F4T: routed rows per expert up to which launches of 8 rows are used (-1 = default)
  int cpt;     // BP_TUNE_CPT: chunks per table pass of the table-lookup GEMV
  int tiles;   // BP_TUNE_TILES: tokens from which bp_moe_layer_* runs its GEMMs over the device-side list of token tiles (-1 = default)
  char glu;    // BP_TUNE_GLU: 'n' bp_moe_layer_* never lets the gate | up GEMM apply SwiGLU itself (a launch of its own instead), 'g' it does but the row gather stays a launch of its own
};
const Tuning& tuning();

// Raises a kernel's dynamic LDS limit, once per device and kernel (thread-safe).
template <auto Kernel>
int raise_lds_limit(int bytes) {
  static std::mutex m;
  static bool done[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(BP_ERR_LAUNCH, "cannot identify the current device");
  std::lock_guard<std::mutex> lock(m);
  if (!done[dev]) {
    const hipError_t rc = hipFuncSetAttribute((const void*)Kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (rc != hipSuccess) return fail(BP_ERR_LAUNCH, "cannot raise the dynamic LDS limit of a kernel: %s", hipGetErrorString(rc));
    done[dev] = true;
  }
  return BP_OK;
}

// Kernel selection for a validated argument block (the body of bp_ternary_grouped_gemm after its checks).
int run_gemm(const GemmArgs& a, hipStream_t s);
// True when a launch in tile-list mode would run on one of the 32-token-tile kernels (which honour tiles / overwrite).
bool gemm_tiles_supported(const GemmArgs& a);
// Workspace bytes of the TQ2 grouped GEMM over converted activations (GemmArgs::stage) for T rows in all; 0: not available.
size_t gemm_tq2f_workspace_bytes(int64_t T, int64_t K, int64_t E);
int launch_general(const GemmArgs& a, hipStream_t s);
// Returns BP_ERR_UNSUPPORTED (without setting an error message) when the shape is outside the
// tuned kernels' preconditions.
int launch_mfma(const GemmArgs& a, hipStream_t s);
bool mfma_supports(const GemmArgs& a);

// ---- device helpers ----
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {  // round to nearest even, NaN kept quiet
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t b) {
  _Float16 h = __builtin_bit_cast(_Float16, b);
  return (float)h;
}

__device__ __forceinline__ float load_scale(const void* p, int dtype, int64_t i) {
  if (dtype == BP_F32) return ((const float*)p)[i];
  const uint16_t b = ((const uint16_t*)p)[i];
  return dtype == BP_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}

__device__ __forceinline__ float load_act_f32(const void* p, int dtype, int64_t i) {
  if (dtype == BP_F32) return ((const float*)p)[i];
  if (dtype == BP_I8) return (float)((const int8_t*)p)[i];
  const uint16_t b = ((const uint16_t*)p)[i];
  return dtype == BP_F16 ? f16_bits_to_f32(b) : bf16_bits_to_f32(b);
}


// TQ1 digit i of byte v as a trit (boilerplate/ternary/pack.py:62-67): bytes >= 243 decode to 0.
__device__ __host__ __forceinline__ int tq1_trit(unsigned v, int i) {
  if (v >= 243u) return 0;
  const unsigned p = i == 0 ? 1u : i == 1 ? 3u : i == 2 ? 9u : i == 3 ? 27u : 81u;
  return (int)((v / p) % 3u) - 1;
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

}  // namespace bp

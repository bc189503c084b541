// C entry point of the grouped ternary GEMM: argument validation (the checks of the reference
// launcher, boilerplate/kernels/csrc/ternary_cuda_kernel.cu:109-141, done without any
// device-to-host copy), kernel selection, and the thread-local error/kernel-name plumbing.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "bp_common.h"
#include "bp_mfma.h"

namespace bp {
namespace {
thread_local char g_error[512] = "";
thread_local char g_kernel[96] = "";
thread_local int g_policy = 0;
}  // namespace

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void note_kernel(const char* name) {
  strncpy(g_kernel, name, sizeof(g_kernel) - 1);
  g_kernel[sizeof(g_kernel) - 1] = 0;
}

void note_kernel_suffix(const char* suffix) {
  const size_t len = strlen(g_kernel);
  if (len + strlen(suffix) + 1 <= sizeof(g_kernel)) strcpy(g_kernel + len, suffix);
}

namespace {
// The overrides in force: an immutable snapshot behind an atomic pointer, so that a launch path on one thread reads a
// consistent set while bp_reload_tuning() on another publishes a new one (old snapshots are never freed: a reader may
// still hold one, and there are only as many as there were reloads).
std::atomic<const Tuning*> g_tuning{nullptr};
std::once_flag g_tuning_once;
void read_tuning() {
  Tuning* t = new Tuning{0, 0, 0, 0, 0, 0, -1, 0, -1, 0};
  if (const char* v = getenv("BP_TUNE_R")) t->r = atoi(v);
  if (const char* v = getenv("BP_TUNE_WAVES")) t->waves = atoi(v);
  if (const char* v = getenv("BP_TUNE_TQ1")) t->tq1 = v[0];
  if (const char* v = getenv("BP_TUNE_TQ2G")) t->tq2g = v[0];
  if (const char* v = getenv("BP_TUNE_TQ2V")) t->tq2v = v[0];
  if (const char* v = getenv("BP_TUNE_F4W")) t->f4w = atoi(v);
  if (const char* v = getenv("BP_TUNE_F4T")) t->f4t = atoi(v);
  if (const char* v = getenv("BP_TUNE_CPT")) t->cpt = atoi(v);
  if (const char* v = getenv("BP_TUNE_TILES")) t->tiles = atoi(v);
  if (const char* v = getenv("BP_TUNE_GLU")) t->glu = v[0];
  g_tuning.store(t, std::memory_order_release);
}
}  // namespace

const Tuning& tuning() {
  std::call_once(g_tuning_once, read_tuning);
  return *g_tuning.load(std::memory_order_acquire);
}

int check_launch(const char* what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(BP_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return BP_OK;
}
}  // namespace bp

using namespace bp;

extern "C" const char* bp_last_error(void) { return g_error; }
extern "C" const char* bp_last_kernel(void) { return g_kernel; }
extern "C" const char* bp_version(void) { return "bp_ternary_hip gfx950"; }

extern "C" void bp_reload_tuning(void) {
  tuning();  // (the first read has happened)
  read_tuning();
}

extern "C" int bp_set_kernel_policy(int policy) {
  const int old = g_policy;
  if (policy >= 0 && policy <= 2) g_policy = policy;
  return old;
}

static bool valid_scale_dtype(int d) { return d == BP_F32 || d == BP_F16 || d == BP_BF16; }
static bool valid_act_dtype(int d) { return d == BP_I8 || d == BP_BF16 || d == BP_F16 || d == BP_F32; }

static int grouped_gemm(float* out, const void* x, int x_dtype, const float* x_scale, const int64_t* offsets,
                        const int64_t* offsets_host, const uint8_t* const* packed, const void* const* w_scale,
                        int scale_dtype, int n_terms, int64_t T, int64_t N, int64_t K, int64_t Kp, int64_t G, int64_t group,
                        int64_t E, int fmt, int64_t max_rows, void* workspace, size_t workspace_bytes, void* stream) {
  g_error[0] = 0;
  g_kernel[0] = 0;
  if (!valid_act_dtype(x_dtype)) return fail(BP_ERR_ARG, "unexpected ternary GEMM activation dtype");
  if (!valid_scale_dtype(scale_dtype)) return fail(BP_ERR_ARG, "unexpected ternary GEMM scale dtype");
  if (fmt != BP_TQ1 && fmt != BP_TQ2) return fail(BP_ERR_ARG, "fmt must be 1 (TQ1) or 2 (TQ2)");
  if (n_terms < 1 || n_terms > BP_MAX_TERMS) return fail(BP_ERR_ARG, "n_terms must be in 1..%d", BP_MAX_TERMS);
  // 127 * group must fit the int32 group accumulator (ternary_cuda_kernel.cu:120-121)
  if (K <= 0 || K > ((int64_t)1 << 40) || group <= 0 || group > ((int64_t)1 << 24))
    return fail(BP_ERR_ARG, "invalid ternary GEMM K or group");
  const int64_t per = fmt == BP_TQ2 ? 4 : 5;
  if (Kp != K / per + (K % per != 0) || G != K / group + (K % group != 0))
    return fail(BP_ERR_ARG, "inconsistent ternary GEMM shapes (Kp or G does not match K)");
  if (T < 0 || N < 0 || E < 0 || T > ((int64_t)1 << 40) || N > ((int64_t)1 << 40))
    return fail(BP_ERR_ARG, "bad output shape");
  if (E > 65535) return fail(BP_ERR_ARG, "too many experts for one launch (grid y limit)");
  if (max_rows < 0) return fail(BP_ERR_ARG, "max_rows must not be negative");
  if (!offsets && E > 0) return fail(BP_ERR_ARG, "offsets must be a device pointer to E + 1 values");
  if (!packed || !w_scale) return fail(BP_ERR_ARG, "null term arrays");
  if (offsets_host) {
    // the reference validates a host copy of the offsets on every call (ternary_cuda_kernel.cu:130-139)
    int64_t widest = 0;
    if (offsets_host[0] != 0 || offsets_host[E] != T)
      return fail(BP_ERR_OFFSETS, "offsets must start at 0 and end at the row count");
    for (int64_t e = 0; e < E; ++e) {
      if (offsets_host[e + 1] < offsets_host[e]) return fail(BP_ERR_OFFSETS, "offsets must be nondecreasing");
      const int64_t w = offsets_host[e + 1] - offsets_host[e];
      if (w > widest) widest = w;
    }
    if (max_rows < widest) return fail(BP_ERR_ARG, "max_rows is smaller than the largest expert row count");
    max_rows = widest;
  }
  if (max_rows > T) max_rows = T;
  if (max_rows == 0 || N == 0 || E == 0 || T == 0) return BP_OK;
  if (!out || !x) return fail(BP_ERR_ARG, "null out or x");
  if (x_dtype == BP_I8 && !x_scale) return fail(BP_ERR_ARG, "int8 activations need x_scale");

  GemmArgs a;
  memset(&a, 0, sizeof(a));
  a.out = out; a.x = x; a.x_scale = x_scale; a.offsets = offsets;
  for (int t = 0; t < n_terms; ++t) {
    if (!packed[t] || !w_scale[t]) return fail(BP_ERR_ARG, "null packed or scale pointer in term %d", t);
    a.packed[t] = packed[t];
    a.w_scale[t] = w_scale[t];
  }
  a.x_dtype = x_dtype; a.scale_dtype = scale_dtype; a.n_terms = n_terms; a.fmt = fmt;
  a.T = T; a.N = N; a.K = K; a.Kp = Kp; a.G = G; a.group = group; a.E = E; a.max_rows = max_rows;
  a.stage = (unsigned char*)workspace;
  a.stage_bytes = workspace ? (int64_t)workspace_bytes : 0;

  return run_gemm(a, (hipStream_t)stream);
}

extern "C" int bp_ternary_grouped_gemm(float* out, const void* x, int x_dtype, const float* x_scale,
                                       const int64_t* offsets, const int64_t* offsets_host,
                                       const uint8_t* const* packed, const void* const* w_scale, int scale_dtype,
                                       int n_terms, int64_t T, int64_t N, int64_t K, int64_t Kp, int64_t G,
                                       int64_t group, int64_t E, int fmt, int64_t max_rows, const int8_t* lut1,
                                       void* stream) {
  (void)lut1;  // the kernels carry the table themselves; see bp_tq1_lut for the tensor form
  return grouped_gemm(out, x, x_dtype, x_scale, offsets, offsets_host, packed, w_scale, scale_dtype, n_terms, T, N, K, Kp, G,
                      group, E, fmt, max_rows, nullptr, 0, stream);
}

static size_t staged_workspace_bytes(int64_t T, int64_t N, int64_t K, int64_t E, int fmt, int64_t max_rows);

extern "C" size_t bp_grouped_gemm_workspace_bytes(int x_dtype, int64_t T, int64_t N, int64_t K, int64_t E, int fmt, int64_t max_rows) {
  if ((fmt != BP_TQ2 && fmt != BP_TQ1) || T <= 0 || E <= 0 || N <= 0 || K <= 0) return 0;
  if (max_rows > T) max_rows = T;
  if (x_dtype == BP_F32 || x_dtype == BP_F16) {  // split into a bf16 pair where only bf16 activations have tuned kernels
    if (K % 256 != 0 || K < 1024 || N % 16 != 0 || (fmt == BP_TQ1 && max_rows == 1)) return 0;
    const size_t pair = 2 * ((((size_t)T * (size_t)K * 2) + 255) & ~(size_t)255);
    return pair + staged_workspace_bytes(T, N, K, E, fmt, max_rows);
  }
  if (x_dtype != BP_BF16) return 0;
  return staged_workspace_bytes(T, N, K, E, fmt, max_rows);
}

static size_t staged_workspace_bytes(int64_t T, int64_t N, int64_t K, int64_t E, int fmt, int64_t max_rows) {
  if (tuning().tq2g == 'b') return 0;
  // (the launcher's own thresholds, so that a call it would turn down does not make its caller allocate)
  if (fmt == BP_TQ2 && tuning().tq2g != 'f' && (N < 1024 || (T + 31) / 32 * ((N + 511) / 512) < 768)) return 0;  // at least two blocks of 512 output rows, three rounds of one workgroup per CU
  if (fmt == BP_TQ1 && max_rows <= 8 && tuning().tq2g != 'f' && !tq1_rows_on_tiles(max_rows, E, T, N)) return 0;  // (the small-batch kernels take these)
  if (max_rows <= 0 || (max_rows + 31) / 32 * 32 * E > 4 * T + 32 * E) return 0;  // a loose bound on the rows per expert: mostly token tiles that do not exist
  return gemm_tq2f_workspace_bytes(T, K, E);
}

extern "C" int bp_ternary_grouped_gemm_ws(float* out, const void* x, int x_dtype, const float* x_scale,
                                          const int64_t* offsets, const int64_t* offsets_host,
                                          const uint8_t* const* packed, const void* const* w_scale, int scale_dtype,
                                          int n_terms, int64_t T, int64_t N, int64_t K, int64_t Kp, int64_t G,
                                          int64_t group, int64_t E, int fmt, int64_t max_rows, void* workspace,
                                          size_t workspace_bytes, void* stream) {
  if (workspace && ((uintptr_t)workspace & 255) != 0) {
    g_error[0] = 0;
    return fail(BP_ERR_ARG, "workspace must be 256-byte aligned");
  }
  return grouped_gemm(out, x, x_dtype, x_scale, offsets, offsets_host, packed, w_scale, scale_dtype, n_terms, T, N, K, Kp, G,
                      group, E, fmt, max_rows, workspace, workspace_bytes, stream);
}

namespace bp {
int kernel_policy() { return g_policy; }

namespace {
// x = hi + lo + e with hi = bf16(x), lo = bf16(x - hi): |e| <= 2^-17 |x| for float32 x; exact for fp16 x (11 significant
// bits: 8 in hi, the other 3 in lo). 8 activations per thread.
template <int XDT>
__global__ __launch_bounds__(256) void k_split_bf16(uint16_t* __restrict__ hi, uint16_t* __restrict__ lo, const void* __restrict__ x, int64_t n8) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
    float v[8];
    if (XDT == BP_F32) {
      const float4 a0 = ((const float4*)x)[2 * i], a1 = ((const float4*)x)[2 * i + 1];
      v[0] = a0.x; v[1] = a0.y; v[2] = a0.z; v[3] = a0.w; v[4] = a1.x; v[5] = a1.y; v[6] = a1.z; v[7] = a1.w;
    } else {
      const uint4 raw = ((const uint4*)x)[i];
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = f16_bits_to_f32((uint16_t)(w[j] & 0xffffu));
        v[2 * j + 1] = f16_bits_to_f32((uint16_t)(w[j] >> 16));
      }
    }
    uint32_t h[4], l[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint16_t h0 = f32_to_bf16_bits(v[2 * j]), h1 = f32_to_bf16_bits(v[2 * j + 1]);
      const uint16_t l0 = f32_to_bf16_bits(v[2 * j] - bf16_bits_to_f32(h0)), l1 = f32_to_bf16_bits(v[2 * j + 1] - bf16_bits_to_f32(h1));
      h[j] = (uint32_t)h0 | ((uint32_t)h1 << 16);
      l[j] = (uint32_t)l0 | ((uint32_t)l1 << 16);
    }
    ((uint4*)hi)[i] = make_uint4(h[0], h[1], h[2], h[3]);
    ((uint4*)lo)[i] = make_uint4(l[0], l[1], l[2], l[3]);
  }
}

// float32 / fp16 activations where only bf16 ones have tuned kernels (TQ2, and TQ1 with more than one token row per
// expert): with a workspace they are split into a bf16 pair and the call runs twice, adding both products into `out`
// (the kernels accumulate). The weights stream twice - against the general kernel's 0.1 TB/s.
bool split_applies(const GemmArgs& a) {
  if (a.x_dtype != BP_F32 && a.x_dtype != BP_F16) return false;
  if (a.fmt == BP_TQ1 && a.max_rows == 1) return false;  // (the single-token TQ1 kernels take these dtypes as they are)
  if (a.tiles || ((uintptr_t)a.x & 15) != 0 || a.K % 8 != 0) return false;
  GemmArgs b = a;
  b.x_dtype = BP_BF16;
  return mfma_supports(b);
}
size_t split_bytes(int64_t T, int64_t K) { return ((size_t)T * (size_t)K * 2 + 255) & ~(size_t)255; }
}  // namespace

int run_gemm(const GemmArgs& a, hipStream_t s) {
  if (g_policy != 1 && a.stage && split_applies(a) && (size_t)a.stage_bytes >= 2 * split_bytes(a.T, a.K)) {
    const size_t part = split_bytes(a.T, a.K);
    uint16_t* hi = (uint16_t*)a.stage;
    uint16_t* lo = (uint16_t*)(a.stage + part);
    const int64_t n8 = a.T * a.K / 8;
    int64_t g = (n8 + 255) / 256;
    if (g > 16384) g = 16384;
    if (a.x_dtype == BP_F32) hipLaunchKernelGGL(k_split_bf16<BP_F32>, dim3((unsigned)g), dim3(256), 0, s, hi, lo, a.x, n8);
    else hipLaunchKernelGGL(k_split_bf16<BP_F16>, dim3((unsigned)g), dim3(256), 0, s, hi, lo, a.x, n8);
    if (const int rc = check_launch("split_bf16")) return rc;
    GemmArgs b = a;
    b.x_dtype = BP_BF16;
    b.stage = a.stage + 2 * part;  // (what is left of the workspace serves the bf16 calls)
    b.stage_bytes = a.stage_bytes - (int64_t)(2 * part);
    if (b.stage_bytes <= 0) { b.stage = nullptr; b.stage_bytes = 0; }
    b.x = hi;
    if (const int rc = run_gemm(b, s)) return rc;
    b.x = lo;
    return run_gemm(b, s);
  }
  if (g_policy != 1 && mfma_supports(a)) {
    const int rc = launch_mfma(a, s);
    if (rc != BP_ERR_UNSUPPORTED) return rc;  // (a tuned variant may turn a launch down, e.g. when its LDS tiles do not fit)
  }
  if (a.tiles) return fail(BP_ERR_UNSUPPORTED, "tile-list mode needs one of the 32-token-tile kernels");
  if (g_policy == 2) return fail(BP_ERR_UNSUPPORTED, "shape is outside the tuned kernels (policy 2 forbids the general kernel)");
  return launch_general(a, s);
}
}  // namespace bp

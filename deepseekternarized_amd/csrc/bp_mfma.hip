// Dispatch of the tuned gfx950 MFMA kernels for group = 128.
#include "bp_mfma.h"

namespace bp {

bool mfma_supports(const GemmArgs& a) {
  // scale groups of 128, or of 256 (two 128-wide work groups per scale) from K = 2048 up
  if ((a.group != 128 && !(a.group == 256 && a.K >= 2048)) || a.N % 16 != 0) return false;
  if (((uintptr_t)a.x & 15) != 0) return false;
  if ((a.max_rows + 15) / 16 > 65535) return false;
  if (a.fmt == BP_TQ2) {
    if (a.x_dtype != BP_BF16 && a.x_dtype != BP_I8) return false;
    if (a.K % 256 != 0 || a.K < 1024) return false;  // whole steps of 64 packed bytes
    // (an odd number of 2-byte scales per row: every other row of scales starts in the middle of a dword, and the kernels
    // read a row's scales in dword-aligned pieces)
    if (a.group == 256 && a.K % 512 != 0 && a.scale_dtype != BP_F32) return false;
    for (int t = 0; t < a.n_terms; ++t) {
      if (((uintptr_t)a.packed[t] & 15) != 0) return false;
      if (((uintptr_t)a.w_scale[t] & 15) != 0) return false;
    }
    return true;
  }
  // TQ1: fp16 / bf16 scales as stored, or float32 ones (the reference's wrappers widen them before the call);
  // bf16 or int8 activations, or any activation dtype for single-token launches
  if (a.scale_dtype != BP_F16 && a.scale_dtype != BP_BF16 && a.scale_dtype != BP_F32) return false;
  if (a.x_dtype != BP_BF16 && a.x_dtype != BP_I8 && a.max_rows != 1) return false;
  if (a.K % 256 != 0 || a.K < 1024) return false;  // whole groups, and an even number of them (4-byte aligned scale rows)
  if (a.group == 256 && a.K % 512 != 0) return false;
  for (int t = 0; t < a.n_terms; ++t)
    if (((uintptr_t)a.w_scale[t] & 3) != 0) return false;
  return true;
}

bool gemm_tiles_supported(const GemmArgs& a) {
  if (!mfma_supports(a) || (a.x_dtype != BP_BF16 && a.x_dtype != BP_I8)) return false;
  if (a.fmt == BP_TQ1) return a.K <= ((int64_t)1 << 24) && a.N * a.Kp <= ((int64_t)1 << 31) - 4096;
  return true;
}

int launch_mfma(const GemmArgs& a, hipStream_t s) {
  if (a.tiles) {  // tile-list mode: only the 32-token-tile kernels read the list
    if (!gemm_tiles_supported(a)) return BP_ERR_UNSUPPORTED;
    return a.fmt == BP_TQ1 ? launch_gemm_tq1(a, s) : launch_gemm_tq2(a, s);
  }
  // rows per wave and waves per workgroup: keep enough workgroups in flight for small problems
  // (an expert without rows exits at once: at most min(E, T) experts do work)
  const int64_t work = (a.E < a.T ? a.E : a.T) * (a.N / 16);
  int R = 1;  // two row sub-tiles per wave cost more registers than they save LDS reads; see BP_TUNE_R
  // 8-wave workgroups run two to a CU, so one's start-up (staging, first loads) overlaps the other's
  // steady state; the TQ2 single-token kernels are light enough on registers for that to win everywhere.
  int waves = work >= 2048 && !(a.fmt == BP_TQ2 && a.max_rows == 1) ? 16 : 8;
  // development overrides (tuning sweeps)
  if (tuning().r == 1 || tuning().r == 2) R = tuning().r;
  if (tuning().waves == 8 || tuning().waves == 16) waves = tuning().waves;
  if (a.fmt == BP_TQ1) return launch_mfma_tq1(a, s, waves);
  if (a.max_rows <= 4) {  // decode GEMV of a large call (up to four token rows per expert): K split over the waves, weights as fp4
    const int rc = launch_tq2_gemv_fp4(a, s);
    if (rc != BP_ERR_UNSUPPORTED) return rc;
  }
  // Experts with more than 16 rows get token tiles of 32 - unless the batch is sparse (on average at most 8 rows per
  // expert) and the bound small: then nearly every expert fits one 16-token tile of the lighter kernel, and the few
  // that do not (or a loose upper bound from a caller that keeps the routing on the device) cost a second tile.
  const bool sparse = a.T <= 8 * a.E && a.max_rows <= 64;
  // A launch of few workgroups (one dense linear on a decode batch: 256 rows x 32 tokens per workgroup leaves most CUs
  // idle) also goes to the 16-token tiles, which make four times as many.
  const bool few = a.E == 1 && ((a.N + 255) / 256) * ((a.max_rows + 31) / 32) < 64 && a.max_rows <= 128;
  if (a.max_rows > 16 && !sparse && !few) return launch_gemm_tq2(a, s);
  return launch_mfma_tq2(a, s, R, 1, waves);
}

}  // namespace bp

/* C ABI of libbp_ternary_hip.so: the gfx950 (MI355X) implementation of Boilerplate's ternary
 * expert-linear path. Plain pointers and sizes only; every pointer marked "device" is HIP device
 * memory on the current device, `stream` is a hipStream_t (NULL = the default stream).
 *
 * Conventions shared by all entry points
 *   - return value 0 = success; anything else is an error code from enum bp_status, and
 *     bp_last_error() then returns a message for the calling thread. The reference's native
 *     boundary raises RuntimeError for every rejected argument
 *     (boilerplate/kernels/csrc/ternary_cuda_kernel.cu:109-141, tests/test_kernel_security.py:25-38);
 *     the Python layer turns a nonzero return into RuntimeError with that message.
 *   - nothing is allocated, freed or retained by the library; launches are asynchronous on `stream`.
 *   - packed weights use the reference layout unchanged (boilerplate/ternary/pack.py:7-16):
 *     row-major [N, Kp] uint8 per expert, Kp = ceil(K/4) (TQ2, fmt 2) or ceil(K/5) (TQ1, fmt 1);
 *     one scale per row per `group` consecutive K entries, [N, G], G = ceil(K/group).
 */
#ifndef BP_TERNARY_H
#define BP_TERNARY_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum bp_status {
  BP_OK = 0,
  BP_ERR_ARG = 1,      /* malformed argument (shape, dtype code, null pointer, range) */
  BP_ERR_OFFSETS = 2,  /* host-visible offsets are not 0-based, nondecreasing and T-terminated */
  BP_ERR_LAUNCH = 3,   /* HIP reported a launch or runtime error */
  BP_ERR_UNSUPPORTED = 4
};

enum bp_dtype {
  BP_I8 = 0,   /* int8 activations with a per-row float32 scale (ternary.ops.quant_act_int8) */
  BP_BF16 = 1,
  BP_F16 = 2,
  BP_F32 = 3
};

enum bp_fmt { BP_TQ1 = 1, BP_TQ2 = 2 }; /* the reference's fmt codes (kernels/ternary_cuda.py:46-49) */

#define BP_MAX_TERMS 4

/* Message of the last error on the calling thread ("" when none). */
const char* bp_last_error(void);

/* Library/ISA identification string, e.g. "bp_ternary_hip gfx950". */
const char* bp_version(void);

/* Grouped (per-expert) ternary GEMM; the dense GEMM/GEMV is the case E = 1.
 *
 *   out[t, n] += x_scale[t] * sum_terms sum_g w_scale[term][e(t), n, g] * sum_{k in g} x[t, k] * trit[term][e(t), n, k]
 *
 * Replaces ternary_grouped_gemm_cuda (boilerplate/kernels/csrc/ternary_cuda_kernel.cu:103-152, bound
 * in ternary_cuda.cpp:7-10) and, for float activations, the CPU twin's float path
 * (boilerplate/kernels/csrc/boilerplate_cpu.cpp:79-128). Differences from the reference signature,
 * all additive: activations may be int8 (x_scale used), bf16, f16 or f32 (x_scale ignored, may be
 * NULL); scales may be f32, f16 or bf16 as stored (ternary/ops.py:37 converts to f32 first);
 * n_terms stacked terms (Mode C, ternary/ops.py:71-79) are summed in one pass over x.
 *
 *   out        device f32 [T, N], accumulated into (the caller zero-fills it, as in the reference)
 *   x          device [T, K] of x_dtype, rows sorted by expert
 *   x_scale    device f32 [T] (required for BP_I8)
 *   offsets    device i64 [E + 1]; expert e owns rows offsets[e] .. offsets[e+1]. Values are clamped
 *              to [0, T] inside the kernels, so malformed device offsets cannot index out of bounds.
 *   offsets_host  optional host copy of offsets (NULL to skip): when given it is validated exactly
 *              like the reference does (start 0, end T, nondecreasing, max_rows >= widest expert)
 *              and a violation returns BP_ERR_OFFSETS. No device-to-host copy is ever made.
 *   packed     host array of n_terms device pointers, each u8 [E, N, Kp]
 *   w_scale    host array of n_terms device pointers, each [E, N, G] of scale_dtype
 *   max_rows   upper bound on offsets[e+1] - offsets[e] (sizes the launch; T is always safe)
 *   lut1       device i8 [256, 5] TQ1 table as produced by bp_tq1_lut / pack.tq1_lut(); may be NULL
 *              (the kernels hold the same table as a constant; when given it is ignored)
 */
int bp_ternary_grouped_gemm(float* out, const void* x, int x_dtype, const float* x_scale,
                            const int64_t* offsets, const int64_t* offsets_host,
                            const uint8_t* const* packed, const void* const* w_scale, int scale_dtype,
                            int n_terms, int64_t T, int64_t N, int64_t K, int64_t Kp, int64_t G,
                            int64_t group, int64_t E, int fmt, int64_t max_rows, const int8_t* lut1,
                            void* stream);

/* bp_ternary_grouped_gemm with a workspace of the caller's (the library allocates no device memory). It has no
 * counterpart in the reference. With a workspace of at least bp_grouped_gemm_workspace_bytes(...) bytes (256-byte
 * aligned device memory; contents undefined before and after the call) the grouped GEMM kernels for bf16 activations
 * (TQ2: more than 16 rows per expert; TQ1: more than 8, and dense batches of 7 or 8) convert the activations to matrix-instruction operands once, in
 * a pass of their own, instead of once per block of output rows; results agree with bp_ternary_grouped_gemm's to
 * float32 rounding of the sums. workspace = NULL, or a size of 0 from bp_grouped_gemm_workspace_bytes (no such kernel
 * for these arguments; a launch too small for it to pay - TQ2: fewer than 1024 output rows, or fewer than 768 blocks
 * of 32 tokens x 512 rows; or max_rows so loose a bound that most of the launch's token tiles would not exist:
 * ceil(max_rows / 32) * 32 * E > 4 T + 32 E, e.g. the default max_rows = T with more than a few experts):
 * identical to bp_ternary_grouped_gemm. T is the row count of x (all experts), max_rows the bound the call will pass.
 * float32 and fp16 activations (the reference CPU kernel's float path, boilerplate/kernels/csrc/boilerplate_cpu.cpp:70-77,
 * 114-124) have tuned kernels only for single-token TQ1 calls; with a workspace every other shape the bf16 kernels cover
 * runs on them as well: the activations are split into a bf16 pair x = hi + lo (exact for fp16, to 2^-17 |x| for float32)
 * and both products are added into out. Without one they run on the general kernel. */
size_t bp_grouped_gemm_workspace_bytes(int x_dtype, int64_t T, int64_t N, int64_t K, int64_t E, int fmt, int64_t max_rows);
int bp_ternary_grouped_gemm_ws(float* out, const void* x, int x_dtype, const float* x_scale,
                               const int64_t* offsets, const int64_t* offsets_host,
                               const uint8_t* const* packed, const void* const* w_scale, int scale_dtype,
                               int n_terms, int64_t T, int64_t N, int64_t K, int64_t Kp, int64_t G,
                               int64_t group, int64_t E, int fmt, int64_t max_rows, void* workspace,
                               size_t workspace_bytes, void* stream);

/* Selects the kernel family for bp_ternary_grouped_gemm on the calling thread:
 *   0 = automatic (tuned kernels where the shape allows, general kernel otherwise)
 *   1 = general kernel only (any K, group, format; int8 path bit-identical to
 *       kernels/ternary_cuda.py:52-64 for one term)
 *   2 = tuned kernels only (BP_ERR_UNSUPPORTED if the shape is not covered)
 * Returns the previous value. */
int bp_set_kernel_policy(int policy);

/* The kernel selection has development overrides (environment variables BP_TUNE_*), read once when the library is first
 * used. This reads them again; it is for tests and tuning sweeps that switch kernels inside one process, and has no
 * counterpart in the reference. Development only: the variables steer which kernel a call runs on (never its result
 * beyond the documented tolerances) and the answer of bp_grouped_gemm_workspace_bytes; a deployment leaves them unset.
 * Safe against launches on other threads: they read either the old or the new set, whole. */
void bp_reload_tuning(void);

/* Name of the kernel the last bp_ternary_grouped_gemm on this thread launched ("" if none). After bp_moe_layer_*: the
 * down projection's kernel, with "+glu", "+gather", "+y16" appended where the gate | up launch applied SwiGLU itself, read
 * its rows through the sort order, and the down launch wrote bf16 rows (diagnostics; the tests read it). */
const char* bp_last_kernel(void);

/* Packed rows -> int8 trits [N, K]; bit-identical to unpack_tq1/unpack_tq2
 * (boilerplate/ternary/pack.py:48-51,73-74): TQ2 code 3 -> +2, TQ1 bytes >= 243 -> 0. */
int bp_unpack_trits(int8_t* trits, const uint8_t* packed, int64_t N, int64_t K, int fmt, void* stream);

/* int8 trits [N, K] -> packed rows [N, Kp]; bit-identical to pack_tq1/pack_tq2
 * (boilerplate/ternary/pack.py:43-45,57-59), pad digit 1. */
int bp_pack_trits(uint8_t* packed, const int8_t* trits, int64_t N, int64_t K, int fmt, void* stream);

/* Stored scales (f16 or bf16) -> float32, elementwise; the conversion of ternary/ops.py:37. */
int bp_expand_scales(float* out, const void* scale, int scale_dtype, int64_t n, void* stream);

/* The reference TQ1 table, [256, 5] int8 (boilerplate/ternary/pack.py:62-67), written to device memory. */
int bp_tq1_lut(int8_t* lut, void* stream);

/* Per-row absmax int8 quantisation (boilerplate/ternary/ops.py:20-25):
 * s = max(amax|x| / 127, 1e-8), q = clamp(rint(x / s), -127, 127). x [M, K] of x_dtype (bf16/f16/f32). */
int bp_quant_act_int8(int8_t* q, float* s, const void* x, int x_dtype, int64_t M, int64_t K, void* stream);

/* BitNet b1.58 absmean quantizer and packer in one kernel: the producer of Mode D weights
 * (absmean_ternary, boilerplate/ternary/fit.py:78-96, followed by pack as in BitLinear.packed_term,
 * boilerplate/qat/bitlinear.py:75-80). Per row and `group` columns: s = scale_dtype(sum |w| / columns in the group)
 * (float32 sum in ascending column order), trit = s > 0 ? clamp(rint(w / s), -1, 1) : 0.
 *   packed  device u8 [N, Kp] in the layout of bp_pack_trits
 *   scale   device [N, G] of scale_dtype (BP_F16 or BP_BF16), G = ceil(K / group)
 *   trits   device i8 [N, K], or NULL when only the packed form is wanted
 *   w       device [N, K] of w_dtype (BP_F32, BP_BF16, BP_F16) */
int bp_absmean_pack(uint8_t* packed, void* scale, int scale_dtype, int8_t* trits, const void* w, int w_dtype,
                    int64_t N, int64_t K, int64_t group, int fmt, void* stream);

/* Stable counting sort of expert ids (boilerplate/kernels/ternary_cuda.py:114-118):
 * order[i] = index of the i-th entry in expert order (ties keep input order), offsets = [0, cumsum(counts)].
 * ids device i64 [n] with values in [0, E) (out-of-range ids are reported through *bad, device i32,
 * set to 1; may be NULL). workspace: device i32 [bp_sort_workspace_ints(n, E)] or NULL when that is 0. */
int64_t bp_sort_workspace_ints(int64_t n, int64_t E);
int bp_sort_by_expert(int64_t* order, int64_t* offsets, const int64_t* ids, int64_t n, int64_t E,
                      int32_t* workspace, int32_t* bad, void* stream);

/* bp_sort_by_expert without a workspace argument and without any allocation. It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc). The per-wave histograms that bp_sort_by_expert takes as `workspace`
 * live in a fixed 4 MiB device array inside the library (one per GPU, held until the process ends), so E is limited
 * to BP_SORT_STATIC_MAX_EXPERTS (more: BP_ERR_ARG). Results are identical to bp_sort_by_expert's. All calls on
 * one GPU share that array: calls that overlap in time on one GPU (different streams) race; calls on one
 * stream are ordered and each clears the counters it uses itself. The first call on a device looks up the array's
 * address and sets a kernel attribute (host-side runtime calls): make it outside any stream capture; later calls
 * on that device are plain kernel launches and can be captured. */
#define BP_SORT_STATIC_MAX_EXPERTS 65536
int bp_sort_by_expert_static(int64_t* order, int64_t* offsets, const int64_t* ids, int64_t n, int64_t E,
                             int32_t* bad, void* stream);

/* The check the reference makes on the host before a grouped launch ("max_rows is smaller than the largest expert row
 * count", boilerplate/kernels/csrc/ternary_cuda_kernel.cu:130-139), for callers that keep the offsets on the device:
 * sets *flag (device i32, cleared by the caller) to 1 if an expert has more than max_rows rows. bp_ternary_grouped_gemm
 * with device offsets computes at most max_rows rows per expert and leaves the others untouched, without an error;
 * max_rows = T is always safe. */
int bp_check_max_rows(int32_t* flag, const int64_t* offsets, int64_t E, int64_t T, int64_t max_rows, void* stream);

/* Row gather dst[i, :] = src[index[i] / divisor, :] (the x[order // k] permute of
 * scripts/eval/ternary_kernel_bench.py:90-93). row_bytes must be a multiple of 2. */
int bp_gather_rows(void* dst, const void* src, const int64_t* index, int64_t divisor, int64_t rows,
                   int64_t src_rows, int64_t row_bytes, void* stream);

/* SwiGLU elementwise stage of an expert MLP (boilerplate/engine/standard.py:151-154):
 * h = bf16(bf16(silu(bf16 gate)) * bf16 up) from the float32 GEMM outputs gate_up [rows, 2*I]
 * (gate in columns [0, I), up in [I, 2I)); h bf16 [rows, I]. */
int bp_swiglu_bf16(void* h, const float* gate, const float* up, int64_t rows, int64_t I, int64_t ld_in, void* stream);

/* Weighted combine of expert outputs (boilerplate/engine/standard.py:173-175):
 * out[token, :] = sum over that token's slots, in ascending expert order, of
 * bf16(bf16(y[pos, :]) * w[token, slot]), accumulated in bf16 like index_add_ on a bf16 tensor.
 * y f32 [T*k, H] in expert-sorted order, inv i64 [T*k] = position of pair (token, slot) in that order,
 * w bf16 [T, k], experts i64 [T, k] (to order the slots of one token), out bf16 [T, H]. */
int bp_moe_combine_bf16(void* out, const float* y, const int64_t* inv, const void* w, const int64_t* experts,
                        int64_t T, int64_t k, int64_t H, void* stream);

/* The router's softmax and top-k (boilerplate/engine/standard.py:160-165: `scores = softmax(logits.float())`,
 * `values, indices = topk(scores, k)`, `values / values.sum()` under norm_topk_prob, `values.to(x.dtype)`), one launch:
 * float32 softmax, the k largest scores per token in descending order with ties to the lower expert id.
 *   weights  device bf16 or f32 [T, k] (weights_dtype BP_BF16 / BP_F32)
 *   experts  device i64 [T, k]
 *   logits   device bf16 / fp16 / f32 [T, E], E <= 1024, k <= 64
 *   renorm   nonzero: the k scores are divided by their sum before rounding */
int bp_route_topk(void* weights, int weights_dtype, int64_t* experts, const void* logits, int logits_dtype, int64_t T, int64_t E,
                  int64_t k, int renorm, void* stream);

/* SwiGLU of the V4 engine's expert MLP (boilerplate/engine/model.py:376-387, `swiglu`): the two linears return bf16,
 * then everything is float32: up clamped to [-limit, limit] and gate to at most limit (limit > 0; 0 = no clamp),
 * silu(gate) * up, times the routing weight when there is one, rounded to bf16 once (the input of w2).
 *   h        device bf16 [rows, I]
 *   gate, up device f32 GEMM outputs, row stride ld_in
 *   weights  device f32 [pairs] routing weights of the (token, slot) pairs, or NULL (a shared expert: no weighting)
 *   order    device i64 [rows]: row r belongs to pair order[r] (bp_sort_by_expert's order), or NULL (row r = pair r) */
int bp_swiglu_v4(void* h, const float* gate, const float* up, const float* weights, const int64_t* order, int64_t pairs,
                 float limit, int64_t rows, int64_t I, int64_t ld_in, void* stream);

/* Combine of the V4 engine's routed experts (boilerplate/engine/model.py:411-420: `y = zeros(float32)`, then for each
 * expert in ascending order `y[idx] += swiglu(...)`, whose results are bf16 and already weighted):
 * out[token, :] = float32 sum over the token's slots, in ascending expert order, of bf16(y[pos, :]);
 * out f32 [T, H] (the caller adds its shared experts and casts, model.py:421-422) or bf16 [T, H] (cast once here). */
int bp_moe_combine_v4(void* out, int out_dtype, const float* y, const int64_t* inv, const int64_t* experts,
                      int64_t T, int64_t k, int64_t H, void* stream);

/* One routed-expert MoE layer after the router's top-k (the per-expert loop of boilerplate/engine/standard.py:156-176,
 * whose experts are TernaryLinear triples, engine/standard.py:37-41 and 151-154): for every (token, slot)
 *   y = down(bf16(bf16(silu(bf16 gate(x))) * bf16 up(x))) * weights[token, slot]       (each linear rounded to bf16)
 *   out[token] = sum of bf16(y) over the token's slots in ascending expert order, accumulated in bf16,
 * as one sort of the routing, one row gather, two grouped launches (gate and up stacked along N), SwiGLU and the
 * combine, all asynchronous on `stream`; nothing is copied to the host and nothing is allocated (capturable in a
 * HIP graph). Beyond 64 tokens the grouped launches run over a device-side list of the 32-row token tiles that exist
 * instead of the reference's `int(offsets.diff().max())` read-back (boilerplate/kernels/ternary_cuda.py:97).
 *   out      device bf16 [T, H]
 *   x        device bf16 [T, H] (16-byte aligned)
 *   experts  device i64 [T, k], values in [0, E), distinct per token (torch.topk indices)
 *   weights  device bf16 [T, k] routing weights
 *   gate_up_packed[t] device u8 [E, 2 I, Kp(H)], gate_up_scale[t] device [E, 2 I, G(H)]: rows [0, I) gate, [I, 2 I) up
 *   down_packed[t]    device u8 [E, H, Kp(I)],   down_scale[t]    device [E, H, G(I)];  n_terms stacked terms each
 *   act      BP_BF16 (activations as they are) or BP_I8 (per-row int8 of every linear's input, boilerplate/ternary/ops.py:20-25)
 *   workspace device memory, 256-byte aligned, at least bp_moe_layer_workspace_bytes(T, H, I, E, k, act, fmt) bytes
 *   bad      device i32 flag set to 1 if an expert id is out of range (may be NULL) */
size_t bp_moe_layer_workspace_bytes(int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int act, int fmt);
int bp_moe_layer_bf16(void* out, const void* x, const int64_t* experts, const void* weights,
                      const uint8_t* const* gate_up_packed, const void* const* gate_up_scale,
                      const uint8_t* const* down_packed, const void* const* down_scale, int scale_dtype,
                      int n_terms, int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int64_t group, int fmt,
                      int act, void* workspace, size_t workspace_bytes, int32_t* bad, void* stream);

/* The same layer with the rounding points of the V4 engine (boilerplate/engine/model.py:376-387 `swiglu`, 407-422 `moe`):
 *   h = bf16(weights[token, slot] * (silu(clamp(float(bf16 gate(x)))) * clamp(float(bf16 up(x)))))   (float32 until the cast)
 *   out[token] = float32 sum of bf16(down(h)) over the token's slots in ascending expert order
 * weights device f32 [T, k] (the router's `weights`, model.py:389-405); swiglu_limit as in the model's config (0: no
 * clamp); out device f32 [T, H] (out_dtype BP_F32: the caller adds the shared experts, which are two more
 * TernaryLinear-style calls, and casts) or bf16 [T, H] (BP_BF16: cast once). Everything else - arguments, workspace
 * (bp_moe_layer_workspace_bytes), no read-back, no allocation - as bp_moe_layer_bf16. */
int bp_moe_layer_v4(void* out, int out_dtype, const void* x, const int64_t* experts, const float* weights, float swiglu_limit,
                    const uint8_t* const* gate_up_packed, const void* const* gate_up_scale,
                    const uint8_t* const* down_packed, const void* const* down_scale, int scale_dtype,
                    int n_terms, int64_t T, int64_t H, int64_t I, int64_t E, int64_t k, int64_t group, int fmt,
                    int act, void* workspace, size_t workspace_bytes, int32_t* bad, void* stream);

/* llama.cpp's TQ1_0 / TQ2_0 blocks (256 weights and one fp16 scale per block; ggml type numbers 34 / 35) from a
 * single-term ternary weight with group 256 and fp16 scales - what the reference makes by dequantizing the weight and
 * calling gguf.quants.quantize on the values (boilerplate/format/gguf_export.py:45-58, 103-114): bit-identical blocks,
 * straight from the packed rows. K must be a multiple of 256, N at most 65535 rows per call.
 *   blocks  device u8 [N, K / 256, bp_gguf_block_bytes(qtype)] (54 bytes for TQ1_0, 66 for TQ2_0)
 *   packed  device u8 [N, Kp] in the layout of bp_pack_trits (fmt), scale device fp16 [N, K / 256] */
#define BP_GGUF_TQ1_0 34
#define BP_GGUF_TQ2_0 35
int64_t bp_gguf_block_bytes(int qtype);
int bp_gguf_from_ternary(uint8_t* blocks, int qtype, const uint8_t* packed, const void* scale, int64_t N, int64_t K,
                         int fmt, void* stream);
/* The other way: such blocks decoded to trits i8 [N, K] (digit - 1) and their scales fp16 [N, K / 256]; bp_pack_trits
 * then gives the packed rows of either format. trit * scale equals gguf.quants.dequantize of the blocks bit for bit
 * (the check of boilerplate/format/gguf_export.py:109-113 and tests/test_gguf_export.py:54-75). */
int bp_gguf_to_trits(int8_t* trits, void* scale, const uint8_t* blocks, int qtype, int64_t N, int64_t K, void* stream);

/* Mode B: canonical-Huffman decode of weight bytes on the device (the device decoder of
 * boilerplate/kernels/csrc/huffman_cuda_kernel.cu:12-79 `huff_decode_into_cuda`; stream layout
 * boilerplate/format/entropy.py:13-18): symbols in blocks of `block`, codes MSB-first back to back, offsets[b] = bit
 * where block b starts (offsets[blocks] = total bits), every block decoded independently through the 2^maxlen-entry
 * table lut[prefix] = (symbol << 8) | length. raw_bytes = 0: out[i] = symbol i (1-byte formats); else out[2 i] =
 * raw[i], out[2 i + 1] = symbol i (2-byte formats: the coded high byte next to the stored low byte).
 *   out, stream, offsets (i64 [blocks + 1]), lut (i32 [2^maxlen]), raw: device memory; stream_bytes >= 4 (padding)
 *   offsets_host / lut_host: optional host copies; when given they are validated exactly as the reference validates
 *       them (huffman_validation.h:16-41), without any device-to-host copy; NULL skips those checks
 *   error   device i32, cleared by the caller: set to 1 when a block's bits are invalid or truncated (where the
 *       reference raises "invalid or truncated Huffman bitstream"); no memory outside the stream, the table and the
 *       output is touched whatever the stream holds. */
int bp_huff_decode(uint8_t* out, int64_t out_bytes, const uint8_t* stream, int64_t stream_bytes, const int64_t* offsets,
                   const int64_t* offsets_host, int64_t n, int64_t block, const int32_t* lut, const int32_t* lut_host,
                   int64_t maxlen, const uint8_t* raw, int64_t raw_bytes, int32_t* error, void* stream_handle);

#ifdef __cplusplus
}
#endif
#endif /* BP_TERNARY_H */

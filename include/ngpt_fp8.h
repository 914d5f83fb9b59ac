/*
 * libngpt_fp8 -- C ABI of the MI355X (gfx950) FP8 contraction path of modded-nanogpt.
 *
 * Every entry point
 *   - takes raw DEVICE pointers, sizes, float scales and a HIP stream (`void* stream` is a
 *     hipStream_t; NULL is the default stream); no torch types cross this boundary;
 *   - only enqueues work on `stream` and returns: no host synchronisation, no allocation, no
 *     pointer is kept after the call.  Scratch memory is passed in by the caller
 *     (`workspace`, sized by the matching *_workspace_bytes function);
 *   - returns 0 on success, a negative NGPT_E* code for an argument error (nothing was
 *     enqueued), or a positive hipError_t if a launch failed.  ngpt_last_error() returns a
 *     thread-local message for the most recent failure.
 *
 * fp8 formats are the OCP ones PyTorch calls float8_e4m3fn (fmt 0) and float8_e5m2 (fmt 1).
 * Scales follow the reference's divide convention: q = x / s, dequantised value = q * s.
 * Weight layout: NGPT_W_OUT_IN = weight stored [N, K] (`nanogpt::mm`),
 *                NGPT_W_IN_OUT = weight stored [K, N] (`nanogpt::mm_t`).
 *
 * File:line citations are relative to the reference checkout (KellerJordan/modded-nanogpt).
 */
#ifndef NGPT_FP8_H
#define NGPT_FP8_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NGPT_OK            0
#define NGPT_EINVAL       -1   /* null pointer / non-positive size */
#define NGPT_EALIGN       -2   /* a dimension violates the stated divisibility rule */
#define NGPT_EWORKSPACE   -3   /* workspace too small */
#define NGPT_ERANGE       -4   /* value outside the supported range (e.g. n_predict, vocab) */

#define NGPT_FMT_E4M3      0
#define NGPT_FMT_E5M2      1

#define NGPT_W_OUT_IN      0
#define NGPT_W_IN_OUT      1

#define NGPT_MAX_PREDICT   4   /* n_predict (multi-token prediction depth) supported by the CE kernels */

int ngpt_abi_version(void);
const char* ngpt_last_error(void);

/* Number of compute units the persistent kernels size their grids to (0 if no device). */
int ngpt_num_cus(void);

/* ---- optional per-kernel timing ------------------------------------------------------------
 * No counterpart in the reference (contributors patch torch.profiler in by hand).  When enabled,
 * the heavy launches of the fused lm_head + CE path are bracketed by HIP events on their own
 * stream.  Slots: 0 fused CE forward kernel, 1 dlogits recompute, 2 dx GEMM, 3 dW GEMM (of the fused CE backward),
 * 4 other fp8 GEMMs, 5 up projection + ReLU^2, 6 dpre, 7 plain bf16 GEMMs of the MLP, 8 MLP input producers.
 * ngpt_profile_read waits for the recorded launches of a slot, returns the sum of their
 * durations and their count, and clears the slot. */
int ngpt_profile_enable(int on);
int ngpt_profile_read(int slot, double* total_ms, int* launches);

#ifdef NGPT_BENCH_BUILD
/* Measurement aids, no counterpart in the reference; they exist only in the measurement build of the library
 * (libngpt_fp8_bench.so, compiled with -DNGPT_BENCH_BUILD), never in libngpt_fp8.so.  That build also accepts
 * out_kind 3 in ngpt_gemm_fp8_tn: the contraction loop alone, result discarded.
 *
 * Microbenchmark of the fp8 GEMM's k-step skeleton (same tile shape and instructions as the tile kernel, no
 * epilogue): one launch of `grid` workgroups x `iters` k-steps of 256 x 256 x 128.  mode bits: 1 = operand fragments
 * re-read from LDS every sub-step, 2 = a workgroup barrier per k-step, 4 = 64 KiB of operands per k-step through
 * direct-to-LDS loads; 0 = the matrix pipe alone.  src: fp8 bytes, 64 KiB + 8 x 64 KiB per workgroup, src_stride
 * bytes apart; sink: 512 floats; ticks [grid][2] int64 = shader-clock cycles and 100 MHz wall ticks per workgroup. */
int ngpt_bench_kstep_rate(const void* src, int64_t src_stride, int mode, int iters, int grid, float* sink,
                          long long* ticks, void* stream);
#endif

/* ---- quantisers ---------------------------------------------------------------------------
 * out[i] = fp8(bf16_rne(fp32(in[i]) / scale)), round-to-nearest-even, NOT saturating
 * (e4m3fn overflow -> NaN code, e5m2 overflow -> +-inf): PyTorch-eager `x.div(s).to(fp8)`.
 * Replaces the inductor-generated quantise kernels behind train_gpt_medium.py:45-46,75 and
 * train_gpt.py:78-79,114, triton_kernels.py:1212-1213.  n % 8 == 0. */
int ngpt_quant_fp8(const void* in_bf16, void* out_f8, int64_t n, float scale, int fmt, void* stream);

/* Same quantiser on a [rows, cols] matrix, writing the row-major copy (out_f8, nullable) and/or
 * the transposed copy out_f8_t [cols, rows] (nullable) in one pass over the input.  Fuses the
 * `.T.contiguous()` copies of train_gpt_medium.py:86-87 / train_gpt.py:129-130 into the
 * quantiser.  rows % 16 == 0, cols % 16 == 0. */
int ngpt_quant_fp8_2d(const void* in_bf16, int rows, int cols, float scale, int fmt,
                      void* out_f8, void* out_f8_t, void* stream);

/* out[c, r] = in[r, c] for 1-byte elements: `transpose_copy` (triton_kernels.py:788-841) for
 * the fp8 operands.  rows % 16 == 0, cols % 16 == 0. */
int ngpt_transpose_u8(const void* in, int rows, int cols, void* out, void* stream);

/* out[c, r] = in[r, c] for elements of 1, 2 or 4 bytes and any shape: `transpose_copy` as the optimizer calls it on
 * the bf16 tied embedding / lm_head weights (train_gpt.py:808-810; triton_kernels.py:788-841). */
int ngpt_transpose_copy(const void* src, int rows, int cols, void* dst, int elem_bytes, void* stream);

/* ---- the GEMM building block --------------------------------------------------------------
 * C[r, c] = scale * sum_k A[r, k] * B[c, k]; A [R, K] and B [C, K] are fp8 with the contraction
 * index contiguous (row strides lda / ldb bytes).  What `torch._scaled_mm` does for the
 * reference (call sites train_gpt_medium.py:47,76,85; train_gpt.py:85,117,128;
 * triton_kernels.py:1217,1268,1283).  out_kind: 0 = bf16, 1 = fp32, 2 = fp32 accumulate
 * (C += ...); 3 = discard the result (times the contraction loop alone) in the measurement build only.  ldc in elements.  K % 128 == 0, lda % 16 == 0, ldb % 16 == 0. */
int ngpt_gemm_fp8_tn(const void* A, int fmt_a, int64_t lda, const void* B, int fmt_b, int64_t ldb,
                     int R, int C, int K, float scale, void* out, int64_t ldc, int out_kind,
                     void* stream);

/* ---- nanogpt::mm / nanogpt::mm_t forward --------------------------------------------------
 * train_gpt_medium.py:40-57 (w_layout OUT_IN, w [N,K]) and train_gpt.py:70-95 (IN_OUT, w [K,N]).
 * x [M,K] bf16.  Writes out [M,N] bf16 = bf16((x_f8 . w_f8^T) * x_s * w_s), x_f8 [M,K] e4m3 and
 * w_f8 (e4m3, same layout as w).  K % 128 == 0, M % 16 == 0, N % 16 == 0.
 * Workspace: IN_OUT needs N x K bytes (the [N, K] copy the GEMM reads).  ngpt_mm_fwd_workspace_bytes adds N x K bytes
 * for N % 64 == 0, K in {256, 512, 768, 1024} and enough tokens to fill the device: with that much the product runs
 * on the token-stationary kernel of the fused cross-entropy (weights in MFMA-fragment order), with less on the tile
 * kernel; same results bit for bit. */
int64_t ngpt_mm_fwd_workspace_bytes(int M, int N, int K, int w_layout);
int ngpt_mm_fwd(const void* x_bf16, const void* w_bf16, int M, int N, int K, float x_s, float w_s,
                void* out_bf16, void* x_f8, void* w_f8, int w_layout,
                void* workspace, int64_t workspace_bytes, void* stream);

/* ---- nanogpt::mm_backward / nanogpt::mm_t_backward ----------------------------------------
 * train_gpt_medium.py:67-95 and train_gpt.py:105-141.  g [M,N] bf16 is quantised to e5m2 with
 * grad_s; dx [M,K] bf16 = (g_f8 . w_f8) * grad_s * w_s; dw_kn [K,N] fp32 contiguous =
 * (x_f8^T . g_f8) * x_s * grad_s.  For OUT_IN the caller exposes dw_kn as its transposed view
 * ([N,K], strides (1,N)), exactly the reference's `.T`.  M % 128 == 0, N % 128 == 0, K % 16 == 0. */
int64_t ngpt_mm_bwd_workspace_bytes(int M, int N, int K, int w_layout);
int ngpt_mm_bwd(const void* g_bf16, const void* x_f8, const void* w_f8, int M, int N, int K,
                float x_s, float w_s, float grad_s, void* dx_bf16, void* dw_kn_f32, int w_layout,
                void* workspace, int64_t workspace_bytes, void* stream);

/* ---- FP8 MLP up-projection with fused ReLU^2 ----------------------------------------------
 * linear_relu_square_kernel FORWARD+USE_FP8(+EMIT_FP8) and its launcher, triton_kernels.py:402-499,
 * 576-665.  x_f8 [M,K] e4m3, w_f8 [N,K] e4m3, dequant: 1-element fp32 DEVICE tensor.
 * post [M,N] bf16 = bf16(max(bf16(acc * *dequant), 0)^2).  If post_f8 != NULL also writes
 * post_f8 [M,N] = e4m3(min(post / *act_scale, 448)) and partial_amax[i] (n_partials fp32 entries;
 * entry i = running max of `post` seen by persistent workgroup i, 0 for unused entries).
 * K % 128 == 0, N % 16 == 0. */
int ngpt_fc_relu2_fwd(const void* x_f8, const void* w_f8, const float* dequant, int M, int N, int K,
                      void* post_bf16, void* post_f8, const float* act_scale,
                      float* partial_amax, int n_partials, void* stream);
/* The same with a workspace of ngpt_fc_relu2_fwd_workspace_bytes (N x K bytes for N % 64 == 0, K in {256, 512, 768,
 * 1024} and enough tokens to fill the device, else 0): the token-stationary kernel of the fused cross-entropy then
 * runs the product (weights re-ordered into the workspace first), with the same results bit for bit.  With post_f8
 * that kernel needs n_partials >= ngpt_num_cus(); otherwise, or without the workspace, the call is
 * ngpt_fc_relu2_fwd. */
int64_t ngpt_fc_relu2_fwd_workspace_bytes(int M, int N, int K);
int ngpt_fc_relu2_fwd_ws(const void* x_f8, const void* w_f8, const float* dequant, int M, int N, int K,
                         void* post_bf16, void* post_f8, const float* act_scale,
                         float* partial_amax, int n_partials, void* workspace, int64_t workspace_bytes, void* stream);

/* The same kernel on bf16 operands (FORWARD without USE_FP8, the reference's DISABLE_FP8 path, launched at
 * triton_kernels.py:716-718): post [M,N] = bf16(max(bf16(x . w^T), 0)^2) for x [M,K], w [N,K] bf16.
 * K % 64 == 0, N % 8 == 0. */
int ngpt_linear_relu2_bf16(const void* x_bf16, const void* w_bf16, int M, int N, int K, void* post_bf16, void* stream);

/* ---- MLP backward through ReLU^2 ----------------------------------------------------------
 * linear_relu_square_kernel with FORWARD = False, triton_kernels.py:472-476, 493-496, called at :726.
 * dy [M, D] bf16, w2 [H, D] bf16, post [M, H] bf16 ->
 * dpre [M, H] = bf16(2 * bf16(dy . w2^T) * sqrt(post)), a bf16 MFMA GEMM (fp32 accumulate) with the
 * product fused into the epilogue.  D % 64 == 0. */
int ngpt_fc_relu2_bwd_dpre(const void* dy_bf16, const void* w2_bf16, const void* post_bf16, int M, int H, int D,
                           void* dpre_bf16, void* stream);

/* ---- the plain bf16 products of the MLP ----------------------------------------------------
 * out[r, c] = bf16(sum_k A(r, k) * B(c, k)), fp32 accumulation, one rounding.  Each operand is a row-major bf16
 * matrix in one of two layouts: NGPT_K_CONTIGUOUS = stored [rows, K] (contraction contiguous, leading dimension
 * >= K), NGPT_K_ROWS = stored [K, rows] (the contraction index is the row, leading dimension >= rows), read
 * through transposing LDS loads without a transposed copy.  Leading dimensions in elements.  Replaces the four
 * cuBLAS products of FusedLinearReLUSquareFunction, triton_kernels.py:715 (`post @ W2`: A = post K_CONTIGUOUS,
 * B = W2 K_ROWS), :723 (`post.T @ grad_output`: both K_ROWS, contraction over the tokens), :727 (`dpre.T @ x`)
 * and :728 (`dpre @ W1`).  Few output tiles with a long contraction are cut along it and meet in fp32.
 * K % 64 == 0, R % 8 == 0, C % 8 == 0.  workspace: ngpt_gemm_bf16_workspace_bytes(R, C, K) bytes. */
#define NGPT_K_CONTIGUOUS  0
#define NGPT_K_ROWS        1
int64_t ngpt_gemm_bf16_workspace_bytes(int R, int C, int K);
int ngpt_gemm_bf16(const void* A, int a_layout, int64_t lda, const void* B, int b_layout, int64_t ldb,
                   int R, int C, int K, void* out_bf16, int64_t ldc, void* workspace, int64_t workspace_bytes,
                   void* stream);

/* ---- fp8 GEMM scaled by two device-resident per-tensor scales --------------------------------
 * out[r, c] = bf16(sum_k A[r, k] * B[c, k] * (*scale_a * *scale_b)), operands fp8 with the contraction contiguous:
 * torch._scaled_mm(post_f8, W2_f8, scale_a=activation_scale, scale_b=W2_scale, out_dtype=bf16), the FP8 down
 * projection of FusedLinearReLUSquareFunction.forward, triton_kernels.py:706-713.  scale_a / scale_b are
 * 1-element fp32 device buffers read by the kernel (no host synchronisation).  K % 128 == 0, C % 4 == 0.
 * workspace: ngpt_gemm_fp8_scaled_workspace_bytes(R, C, K) bytes (tiles cut along a long contraction meet in fp32). */
int64_t ngpt_gemm_fp8_scaled_workspace_bytes(int R, int C, int K);
int ngpt_gemm_fp8_scaled(const void* A, int fa, int64_t lda, const void* B, int fb, int64_t ldb, int R, int C, int K,
                         const float* scale_a, const float* scale_b, void* out_bf16, int64_t ldc,
                         void* workspace, int64_t workspace_bytes, void* stream);

/* ---- delayed-scaling bookkeeping of the FP8 down projection, tied-embedding gradient add -----
 * scales[l] = max(max_i partial_amax[l * partial_stride + i], 1e-12) * headroom / 448:
 * reduce_mlp_activation_scales(_kernel), triton_kernels.py:502-519, 732-745. */
int ngpt_reduce_scales(const float* partial_amax, int64_t partial_stride, int num_layers, int partial_count,
                       float headroom, float* scales, void* stream);

/* The tile kernel of quantize_transpose_mlp_down_weights, triton_kernels.py:522-565, 748-778:
 * weights [L, hidden, model_dim] bf16 (layer stride in elements) -> out_f8 [L, model_dim, hidden] =
 * e4m3(clamp(w / scales[l], +-448)); used_scales[l] = scales[l]; partial_amax[l, tile] = max |w| over
 * each 64 x 64 tile (tiles = ceil(hidden/64) * ceil(model_dim/64)).  The caller then reduces the
 * partials into the next scales with ngpt_reduce_scales.  hidden % 16 == 0, model_dim % 16 == 0. */
int ngpt_quant_transpose_down(const void* weights_bf16, int num_layers, int hidden, int model_dim,
                              int64_t layer_stride, const float* scales, void* out_f8, float* used_scales,
                              float* partial_amax, void* stream);

/* MLP input producer, train_gpt.py:1643-1647 with norm() = F.rms_norm(x, (dim,)) (:952-953):
 *   normed  = rms_norm(x)                         bf16 [rows, dim]
 *   amax    = max(|normed|) clamped to 1e-12      (bf16 value)
 *   x_f8    = e4m3(bf16(normed * q)),  q = bf16(bf16(1 / amax) * 448)   (eager: `448.0 / amax` is amax.reciprocal() * 448.0)
 *   dequant = up_scale[0] * amax / 448            1-element fp32 device buffer (no host sync)
 * Two passes over the activations.  up_scale and dequant are device pointers.  dim % 8 == 0, dim <= 2048.
 * workspace: ngpt_mlp_input_quant_workspace_bytes() bytes of device memory. */
int64_t ngpt_mlp_input_quant_workspace_bytes(void);
int ngpt_mlp_input_quant(const void* x_bf16, int rows, int dim, const float* up_scale, void* normed_bf16,
                         void* x_f8, float* dequant, void* workspace, int64_t workspace_bytes, void* stream);

/* Backward of the norm inside ngpt_mlp_input_quant: dx = d/dx [ F.rms_norm(x, (dim,)) ] . g for bf16 x, g
 * [rows, dim], fp32 arithmetic, one rounding to bf16 (the reference leaves this to autograd through
 * `norm`, train_gpt.py:952-953 and 1643).  dim % 8 == 0, dim <= 2048. */
int ngpt_rmsnorm_bwd(const void* x_bf16, const void* g_bf16, int rows, int dim, void* dx_bf16, void* stream);

/* Up-projection part of GPT.quantize_mlp_fp8, train_gpt.py:1419-1422: per layer l of w [layers, per_layer] bf16,
 *   scales[l] = bf16(max(amax(|w_l|), 1e-12) / 448)   (written as fp32)
 *   w_f8[l]   = e4m3(bf16(w_l / scales[l]))
 * per_layer % 8 == 0.  workspace: ngpt_quant_up_weights_workspace_bytes(layers) bytes. */
int64_t ngpt_quant_up_weights_workspace_bytes(int layers);
int ngpt_quant_up_weights(const void* w_bf16, int layers, int64_t per_layer, void* w_f8, float* scales,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* dst [cols, rows] += src [rows, cols]^T for bf16 (elem_bytes 2) or fp32 (4):
 * transpose_add, triton_kernels.py:844-903. */
int ngpt_transpose_add(const void* src, int rows, int cols, void* dst, int elem_bytes, void* stream);

/* ---- nanogpt::ce_fwd_bwd on materialised logits -------------------------------------------
 * ce_fwd_bwd_kernel, triton_kernels.py:956-1170, 1182-1206.  logits [n_rows, n_cols] bf16,
 * targets/prefix_targets int64 [n_rows], mtp_weights fp32 [n_predict], prefix_weight fp32 [1].
 * prefix_targets / prefix_weight may be NULL (no prefix term).
 * Writes losses fp32 [n_rows] and grad e5m2 [n_rows, n_cols] (saturating store).
 * n_cols % 8 == 0, 1 <= n_predict <= NGPT_MAX_PREDICT.  The workspace holds two lookup
 * tables over the bf16 logit values. */
/* Host-only check (no GPU work, callable without a device): can the CE kernels evaluate the softcap
 * A * sigmoid((l + B) / C) for these constants?  Their lookup tables cover bf16 logits with |l| in [2^-12, 2^8)
 * exactly and assume that sigma no longer changes outside, and they sum exponentials relative to the cap A.
 * Returns NGPT_OK (the reference's 23 / 5 / 7.5 and e.g. 30 / 0 / 7.5, the 15 * tanh(x / 15) + 15 form of
 * train_gpt.py:1683-1684) or NGPT_ERANGE with a message.  The three CE entry points below apply the same
 * check and return NGPT_ERANGE instead of a silently wrong loss. */
int ngpt_softcap_supported(float A, float B, float C);

int64_t ngpt_ce_fwd_bwd_workspace_bytes(void);
int ngpt_ce_fwd_bwd(const void* logits_bf16, const int64_t* targets, const float* mtp_weights,
                    const int64_t* prefix_targets, const float* prefix_weight,
                    float* losses, void* grad_e5m2, int n_rows, int n_cols, int n_predict,
                    float A, float B, float C, float grad_s, float grad_scale,
                    void* workspace, int64_t workspace_bytes, void* stream);

/* ---- fused lm_head + softcapped cross-entropy ---------------------------------------------
 * FusedSoftcappedCrossEntropy.forward/backward, triton_kernels.py:1208-1292, without the
 * [M, V] logits ever being stored: the forward keeps per-row softmax statistics from vocabulary
 * tiles; the backward rebuilds the e5m2 gradient of the logits -- from recomputed logits
 * (ngpt_lmhead_ce_bwd) or from one code byte per logit kept by the forward (the _codes pair) --
 * and does store that gradient, once, in its workspace (M x V bytes) as the operand of dx and dW.
 *
 * Forward: x [M,K] bf16, w bf16 in `w_layout` ([V,K] or [K,V]).  Writes losses [M] fp32 and,
 * saved for backward: lse [M] fp32 (log-sum-exp of the softcapped logits), saved_sigma
 * [(NGPT_MAX_PREDICT + 1) * M] fp32 (the bf16-rounded sigmoid at every candidate target column;
 * entries of invalid targets are zero), x_f8 [M,K] and w_f8_vk [V,K] (e4m3, always
 * vocabulary-major).  K % 128 == 0, M % 16 == 0, V % 16 == 0.
 * Two kernels serve the forward.  For V % 64 == 0 and K in {256, 512, 768, 1024} a token-stationary
 * kernel keeps 128 tokens' activations in LDS and streams the weights from a second, MFMA-fragment
 * ordered copy that lives in the workspace (V x K bytes); ngpt_lmhead_ce_fwd_workspace_bytes
 * includes it.  A workspace of only ngpt_lmhead_ce_fwd_min_workspace_bytes (lookup tables and
 * partial sums) selects the generic tile kernel, as do all other shapes.  Results agree to the
 * last bits of the sum of exponentials (different summation order); codes and fp8 copies are equal. */
int64_t ngpt_lmhead_ce_fwd_workspace_bytes(int M, int K, int V, int w_layout);
int64_t ngpt_lmhead_ce_fwd_min_workspace_bytes(int M, int K, int V, int w_layout);
int ngpt_lmhead_ce_fwd(const void* x_bf16, const void* w_bf16, const int64_t* targets,
                       const float* mtp_weights, int n_predict,
                       const int64_t* prefix_targets, const float* prefix_weight,
                       int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                       float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                       int w_layout, void* workspace, int64_t workspace_bytes, void* stream);

/* The same forward for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no workspace argument, the library uses a buffer of its own that
 * is part of its code object (a static device array of about 1.1 MB, held by every GPU the library runs on
 * until the process ends).  It has no counterpart in the reference.  Arguments and results are those of
 * ngpt_lmhead_ce_fwd; M may be at most ngpt_lmhead_ce_fwd_static_max_rows() (65536), more is NGPT_ERANGE.
 * The call allocates and frees nothing.  All calls on one GPU share that GPU's buffer: calls that may overlap
 * on one GPU (two streams, two host threads) race; issue them on one stream or use ngpt_lmhead_ce_fwd. */
int ngpt_lmhead_ce_fwd_static_max_rows(void);
int ngpt_lmhead_ce_fwd_static(const void* x_bf16, const void* w_bf16, const int64_t* targets,
                              const float* mtp_weights, int n_predict,
                              const int64_t* prefix_targets, const float* prefix_weight,
                              int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                              float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                              int w_layout, void* stream);

/* Backward: gradients of sum(losses) * grad_scale (the incoming autograd gradient is ignored,
 * as in triton_kernels.py:1117,1262).  dx [M,K] bf16; dw fp32 in the weight's own layout
 * ([V,K] for OUT_IN, [K,V] for IN_OUT).  M % 128 == 0, V % 128 == 0, K % 128 == 0. */
int64_t ngpt_lmhead_ce_bwd_workspace_bytes(int M, int K, int V, int w_layout);
int ngpt_lmhead_ce_bwd(const void* x_f8, const void* w_f8_vk, const int64_t* targets,
                       const float* mtp_weights, int n_predict,
                       const int64_t* prefix_targets, const float* prefix_weight,
                       const float* lse, const float* saved_sigma, int M, int K, int V,
                       float x_s, float w_s, float grad_s, float grad_scale,
                       float A, float B, float C, void* dx_bf16, void* dw_f32, int w_layout,
                       void* workspace, int64_t workspace_bytes, void* stream);

/* The same pair with the softcap's output kept between them instead of recomputed (what FusedSoftcappedCrossEntropy
 * saves between forward and backward is one byte per logit either way: the reference keeps the e5m2 gradient,
 * triton_kernels.py:1231-1253, this pair keeps an 8-bit code of bf16(sigmoid(..)), never the logits).  The forward
 * also writes sigma_codes, ngpt_lmhead_ce_codes_bytes(M, V) bytes; the backward turns them into the e5m2 gradient
 * (bit-identical to what ngpt_lmhead_ce_bwd recomputes) without running the logits GEMM a second time.  A sigma below
 * the 255 codes' range (logits under about -13 with A, B, C = 23, 5, 7.5) reads as a zero gradient where that is exact
 * (the row's factor is small enough for every such gradient to round to zero in e5m2); the 256 x 256 tiles of the logits
 * where it is not are listed on the device and recomputed as ngpt_lmhead_ce_bwd does, so results never depend on the range.
 * Everything else (arguments, alignment, workspaces) is as in ngpt_lmhead_ce_fwd / ngpt_lmhead_ce_bwd. */
int64_t ngpt_lmhead_ce_codes_bytes(int M, int V);
int ngpt_lmhead_ce_fwd_codes(const void* x_bf16, const void* w_bf16, const int64_t* targets,
                             const float* mtp_weights, int n_predict,
                             const int64_t* prefix_targets, const float* prefix_weight,
                             int M, int K, int V, float x_s, float w_s, float A, float B, float C,
                             float* losses, float* lse, float* saved_sigma, void* x_f8, void* w_f8_vk,
                             void* sigma_codes, int w_layout, void* workspace, int64_t workspace_bytes, void* stream);
int ngpt_lmhead_ce_bwd_codes(const void* x_f8, const void* w_f8_vk, const int64_t* targets,
                             const float* mtp_weights, int n_predict,
                             const int64_t* prefix_targets, const float* prefix_weight,
                             const float* lse, const float* saved_sigma, const void* sigma_codes, int M, int K, int V,
                             float x_s, float w_s, float grad_s, float grad_scale,
                             float A, float B, float C, void* dx_bf16, void* dw_f32, int w_layout,
                             void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NGPT_FP8_H */

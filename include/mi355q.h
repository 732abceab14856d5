/*
 * mi355q -- C ABI of the MI355X (gfx950) quantized-linear kernels.
 *
 * Every entry point takes raw device pointers, explicit sizes and a HIP
 * stream (passed as void*, it is a hipStream_t; NULL = the null stream),
 * enqueues its work asynchronously on that stream and returns 0 on success
 * or a non-zero code; mi355q_last_error() then describes the failure
 * (thread-local).  Nothing here synchronises with the host and nothing
 * allocates device memory: every output and workspace belongs to the caller.
 *
 * Each declaration names the operator of the reference (EnflameTechnology/
 * vllm-gcu) whose vendor-library call it replaces.
 */
#ifndef MI355Q_H
#define MI355Q_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of activations / outputs */
enum { MI355Q_F16 = 0, MI355Q_BF16 = 1, MI355Q_F32 = 2 };

/* how zero-points are handed to the W4A16 kernels */
enum {
  MI355Q_ZP_NONE = 0,      /* symmetric int4: z = 8 everywhere                      */
  MI355Q_ZP_PACKED = 1,    /* int32 [K/g, N/8], nibble j of column c = z[g, 8c+j]   */
  MI355Q_ZP_PRESCALED = 2  /* activation-dtype [K/g, N] holding z*scale (the form   */
                           /* the reference's GPTQ loader produces,                 */
                           /* vllm_gcu/kernels/quantization/rearrange.py:33-34)     */
};

/* source formats understood by the int4 repack kernels */
enum {
  MI355Q_W4_SRC_GPTQ = 0,      /* int32 [K/8, N], nibble i of row r = k 8r+i (rearrange.py:13-21)     */
  MI355Q_W4_SRC_AWQ = 1,       /* int32 [K, N/8], AWQ interleave (rearrange.py:66-95)                 */
  MI355Q_W4_SRC_REF_KN = 2,    /* uint8 [K/2, N] reference half-group layout (rearrange.py:36-56)     */
  MI355Q_W4_SRC_REF_NK = 3,    /* uint8 [N, K/2] the same, stored transposed for MoE experts          */
  MI355Q_W4_SRC_REF_KN_G64S = 4 /* int8 [K/2, N], half-groups of 32 rows, nibbles hold w - 8 (the w4a8
                                  experts: rearrange.py:61-133 with use_w4a8, rearrange_group 64, as
                                  vllm_gcu/kernels/quantization/w4a8.py:134-220 stores them)          */
                               /* (vllm_gcu/kernels/quantization/moe_wna16.py:464-466)                */
};

const char* mi355q_last_error(void);
int mi355q_abi_version(void);

/* ---- int4 weight formats (load time) ------------------------------------
 * Replaces the CPU repack of rearrange_uint4_int32_uint8_gptq / _awq
 * (vllm_gcu/kernels/quantization/rearrange.py:6-133) by device kernels that
 * produce this library's slab layout: int32 [K/8, N] flat stream
 * [N/128][K/128][8 tiles][64 lanes][4 words]; word s of lane l (c = l%16,
 * kq = l/16) of tile t holds, in nibble {0,4,1,5,2,6,3,7}[j], the weight at
 * k = 128g + 32s + 8kq + j, n = 128S + 8c + t.  K and N must be multiples of
 * 128.  `batch` matrices are converted back to back (MoE experts). */
int mi355q_w4_repack(const void* src, int src_format, int32_t* dst,
                     int batch, int K, int N, void* stream);
/* zero-points -> MI355Q_ZP_PACKED.  src_format GPTQ: int32 [G, N/8] with the
 * "+1" convention (rearrange.py:24-29); AWQ: int32 [G, N/8] interleaved
 * (rearrange.py:96-101). */
int mi355q_w4_repack_zeros(const int32_t* src, int src_format, int32_t* dst,
                           int batch, int G, int N, void* stream);
/* debug / parity: slab layout -> uint8 [K, N] (one value per byte) */
int mi355q_w4_unpack(const int32_t* packed, uint8_t* dst, int batch, int K, int N,
                     void* stream);

/* ---- W4A16 GEMM ----------------------------------------------------------
 * Replaces topsatenGemmQuant as called by gptq_gemm_gcu / awq_gemm_gcu
 * (csrc/src/gptq_gemm_gcu.cpp:27-48, csrc/src/awq_gemm_gcu.cpp:27-47):
 *   out[M, N] = x[M, K] @ ((q - z) * s)[K, N] (+ bias[N]),  fp32 accumulate.
 * x, out, scales, bias share `dtype` (F16 or BF16); qweight is the slab
 * layout; scales [K/g, N]; group_size a multiple of 32 dividing K that divides
 * 128 or is a multiple of it (or -1 for one group).  M <= 64 runs the split-K
 * streaming kernel, larger M the LDS-staged MFMA kernels (groups of 32, 64 and
 * multiples of 128; other sizes go through the streaming kernel 32 rows at a
 * time), which split K over two kernels when their grid would leave most of
 * the chip idle.  bf16 activations of 65 rows or more on outputs of about two million
 * elements or more are first stored in the workspace as fp16 rows, each times a
 * power of two of its own (exact), and take the fp16 kernels (group sizes that
 * are multiples of 128, zero-points not pre-scaled); with a workspace too small
 * for that the bf16 kernel runs (same tolerance, other bits).
 * `workspace` must hold
 * mi355q_w4a16_workspace_bytes() bytes, be zero-filled once before first use,
 * and must not be shared by launches that may overlap in time. */
size_t mi355q_w4a16_workspace_bytes(int M, int K, int N);
int mi355q_w4a16_gemm(void* out, const void* x, const int32_t* qweight,
                      const void* scales, const void* zeros, int zeros_kind,
                      const void* bias, int M, int K, int N, int group_size,
                      int dtype, void* workspace, size_t workspace_bytes,
                      void* stream);
/* tuning hook used by the benchmark.  split_k: bits 0..7 force the split-K
 * factor, bits 8..15 the tiles (of 16 columns) per workgroup of the streaming
 * kernel (1, 2, 4 or 8); 0 in a field = automatic.  family: 0 = auto,
 * 1 = streaming, 2 = MFMA tiles of 64 rows (32 x 64 below 129 rows on narrow
 * layers), 3 = MFMA workgroups of up to 128 rows fed through a ring of LDS
 * stages (fp16, group sizes that are multiples of 128; there bits 8..15 of
 * split_k = 1 or 4 select workgroups of 128 or 512 columns instead of
 * 256; bf16 above 64 rows with the full workspace: the rows staged as
 * fp16, workgroups of 256 or 512 columns). */
int mi355q_w4a16_gemm_ex(void* out, const void* x, const int32_t* qweight,
                         const void* scales, const void* zeros, int zeros_kind,
                         const void* bias, int M, int K, int N, int group_size,
                         int dtype, void* workspace, size_t workspace_bytes,
                         int split_k, int family, void* stream);

/* No counterpart in the reference (the vendor GEMM chooses its own launch).  The work split the streaming
 * kernel takes for M <= 64 rows of a shape on the current device: 16-column tiles per workgroup (1, 2, 4
 * or 8) and the number of K ranges that separate workgroups sum through the workspace. */
int mi355q_w4a16_stream_plan(int M, int K, int N, int group_size, int* tiles_per_workgroup, int* k_splits);

/* No counterpart in the reference.  mi355q_w4a16_gemm for callers that cannot allocate device memory
 * or pass a workspace (code under HIP graph capture, serving loops and harnesses that forbid
 * allocation): same arguments without the workspace, same kernels, bit-identical results (but for
 * bf16 inputs tall enough for mi355q_w4a16_gemm to stage them as fp16 rows in its workspace: the
 * fixed array has no room for that, the bf16 kernel runs here -- same tolerance, other bits).  The
 * split-K partial tiles and arrival counters live in a fixed array of
 * mi355q_w4a16_noalloc_scratch_bytes() = 32 MiB of device memory that every GPU running the library
 * holds until the process ends.  A shape whose split-K plan needs more is rejected with an error
 * (use mi355q_w4a16_gemm then).  All calls on one GPU share the array: calls that may overlap in time
 * on one GPU (different streams, different threads) race and must be serialised by the caller.
 * Calls no allocating routine; enqueues one small clearing kernel before a split-K launch (after every
 * argument check).  The first call on a device looks the array's address up (hipGetSymbolAddress):
 * make one call on each device before capturing a graph that contains this entry point. */
size_t mi355q_w4a16_noalloc_scratch_bytes(void);
int mi355q_w4a16_gemm_noalloc(void* out, const void* x, const int32_t* qweight, const void* scales,
                              const void* zeros, int zeros_kind, const void* bias, int M, int K, int N,
                              int group_size, int dtype, void* stream);

/* fp8-e4m3 block-scaled GEMM for prefill-sized M: the arithmetic of linear_quant
 * (csrc/src/linear_quant.cpp:16-95; vllm_gcu/kernels/quantization/fp8.py:169-205) on an MFMA
 * tile kernel,
 *   out[m, n] = sum_kb x_scale[m, kb] * w_scale[n / 128, kb] * (sum over K block kb of x[m, k] * w[n, k]) (+ bias[n])
 * x is [M, K] fp8 with row stride ldx bytes and scales f32 [M, K/128]; w is [N, K] fp8 with row
 * stride ldw bytes, or in the kslab order when ldw = 0 (see mi355q_kslab_repack), scales f32
 * [N/128, K/128]; bias in the output dtype (f16 / bf16) or NULL.  K %% 128 == 0, N %% 128 == 0.
 * mi355q_kcontig_gemm (quant_mode 1) computes the same and is the faster one up to about 128 rows. */
int mi355q_fp8_block_gemm(void* out, const void* x, const void* w, const float* x_scale,
                          const float* w_scale, const void* bias, int M, int N, int K, long ldx,
                          long ldw, long ldo, int out_dtype, void* stream);

/* fp8-e4m3 GEMM with the scales outside the K sum: what cutlass_scaled_mm computes when it is handed
 * fp8 operands (csrc/src/cutlass_scaled_mm.cpp:12-36 forwards any dtype to topsatenDotBiasQuant with
 * x_scale 0-d -> [1] and w_scale [N, 1] -> [N]; reached from the non-block branch of
 * Fp8GCULinearMethod.apply, vllm_gcu/kernels/quantization/fp8.py:68-69),
 *   out[m, n] = (sum_k x[m, k] * w[n, k]) * x_scale[m or 0] * w_scale[n or 0] (+ bias[n]),   fp32 accumulation.
 * x is [M, K] fp8 with row stride ldx bytes; w is [N, K] fp8 with row stride ldw bytes, or in the
 * kslab order when ldw = 0; x_scale f32 [M] when x_scale_per_row else one value; w_scale f32 [N]
 * when w_scale_per_col else one value; bias in the output dtype (f16 / bf16) or NULL; out row
 * stride ldo elements.  K %% 128 == 0, N %% 4 == 0.  Up to 64 rows (and for layers with few
 * 256 x 128 output tiles) the weight-streaming kernel runs and wants dense operands
 * (ldx = K, ldw = K or 0, ldo = N); above, the MFMA tile kernel (N %% 128 == 0, strides multiples of 16). */
int mi355q_fp8_scaled_gemm(void* out, const void* x, const void* w, const float* x_scale,
                           int x_scale_per_row, const float* w_scale, int w_scale_per_col,
                           const void* bias, int M, int N, int K, long ldx, long ldw, long ldo,
                           int out_dtype, void* stream);
/* The two fp8 GEMMs with a workspace (no counterpart in the reference: the vendor GEMM chooses its own
 * launch).  A layer with few 256 x 128 output tiles behind a long K leaves most of the chip idle; with
 * mi355q_fp8_gemm_workspace_bytes(M, N, K) bytes (0 = this shape is not split; below 65 rows it is not 0
 * only where the split launch is ahead of the weight-streaming kernel) K is cut into ranges of
 * whole K blocks that run side by side, and a second launch adds their fp32 sums in range order and
 * applies bias (and, for the scaled GEMM, the scales): run-to-run identical, and equal to the unsplit
 * launch up to the order of the fp32 additions.  The workspace follows the rules of
 * mi355q_w4a16_gemm's (its first MiB is left alone); without one, or with a smaller one, the unsplit
 * launch (or, for the scaled GEMM on few tiles, the streaming kernel) runs.
 * mi355q_fp8_block_gemm_ws also uses ceil16(M) * (K / 128) * 4 bytes behind the partial sums (behind the first
 * MiB where nothing is split), when the workspace has them, on layers of 128 column tiles or 384 output tiles
 * and more: the activation scales re-ordered K block major by a small launch of its own, so that a workgroup's
 * 256 scales of a K block are 1 KiB in a row instead of one value per cache line.  Same output bits. */
size_t mi355q_fp8_gemm_workspace_bytes(int M, int N, int K);
int mi355q_fp8_block_gemm_ws(void* out, const void* x, const void* w, const float* x_scale,
                             const float* w_scale, const void* bias, int M, int N, int K, long ldx,
                             long ldw, long ldo, int out_dtype, void* workspace, size_t workspace_bytes,
                             void* stream);
int mi355q_fp8_scaled_gemm_ws(void* out, const void* x, const void* w, const float* x_scale,
                              int x_scale_per_row, const float* w_scale, int w_scale_per_col,
                              const void* bias, int M, int N, int K, long ldx, long ldw, long ldo,
                              int out_dtype, void* workspace, size_t workspace_bytes, void* stream);

/* ---- W8A8 int8 -------------------------------------------------------------
 * Replaces topsatenDotBiasQuant as called by cutlass_scaled_mm
 * (csrc/src/cutlass_scaled_mm.cpp:12-36) and dot_bias_quant
 * (csrc/src/dot_bias_quant.cpp:12-24):
 *   out[m, n] = (sum_k x[m, k] * w[n, k]  in int32) * x_scale[m or 0] * w_scale[n or 0] (+ bias[n])
 * x is [M, K] int8 with row stride ldx bytes; w is [N, K] int8 (K contiguous)
 * with row stride ldw bytes -- the physical layout of a checkpoint's [N, K]
 * weight, i.e. the `weight.t()` view the compressed-tensors path passes; ldw = 0
 * says that w is in the kslab order instead (see mi355q_kslab_repack; N % 64 == 0),
 * the layout mi355q_kcontig_gemm streams fastest at decode-sized M.
 * Scale pointers may be NULL (= 1.0); *_per_row / *_per_col select a vector
 * or a single value.  bias is in the output dtype, or fp32 when bias_f32.
 * acc_out (optional) receives the raw int32 accumulators [M, N] for parity
 * checks.  K %% 128 == 0, N %% 4 == 0. */
int mi355q_w8a8_int8_gemm(void* out, int32_t* acc_out, const int8_t* x, const int8_t* w,
                          const float* x_scale, int x_scale_per_row, const float* w_scale,
                          int w_scale_per_col, const void* bias, int bias_f32, int M, int N, int K,
                          long ldx, long ldw, long ldo, int out_dtype, void* stream);
/* The same with a workspace (no counterpart in the reference: the vendor GEMM chooses its own launch).
 * A layer with few 256 x 128 output tiles (N of 4096 .. 10240 at up to a few hundred rows) leaves
 * most of the chip idle behind a long K; with mi355q_w8a8_int8_workspace_bytes(M, N, K) bytes of
 * workspace (0 = this shape is not split) K is cut into ranges that run side by side, and a second
 * launch adds their int32 sums and applies the scales and the bias: integer sums, so the result --
 * acc_out included -- is bit for bit that of the call without workspace.  The workspace follows the
 * rules of mi355q_w4a16_gemm's (its first MiB is left alone, so one buffer serves both); without
 * one, or with a smaller one, the unsplit launch runs. */
size_t mi355q_w8a8_int8_workspace_bytes(int M, int N, int K);
int mi355q_w8a8_int8_gemm_ws(void* out, int32_t* acc_out, const int8_t* x, const int8_t* w,
                             const float* x_scale, int x_scale_per_row, const float* w_scale,
                             int w_scale_per_col, const void* bias, int bias_f32, int M, int N, int K,
                             long ldx, long ldw, long ldo, int out_dtype, void* workspace,
                             size_t workspace_bytes, void* stream);
/* Replaces topsvllmDynamicScaledInt8Quant (csrc/src/dynamic_scaled_int8_quant.cpp:12-19):
 * per row scale = absmax / 127 (fp32 [M]), q = sat_s8(rne(x * (127 / absmax))).
 * valid_rows (optional device int32[1]) limits the rows processed. */
int mi355q_dynamic_int8_quant(int8_t* out, float* scales, const void* x, int M, int K, int dtype,
                              const int32_t* valid_rows, void* stream);
/* Replaces topsatenQuantize as called by static_scaled_int8_quant
 * (csrc/src/static_scaled_int8_quant.cpp:12-28): q = sat_s8(rne(x * (1/scale)))
 * with the reciprocal rounded to the input dtype; scale is one value or [K]. */
int mi355q_static_int8_quant(int8_t* out, const void* x, const float* scale, int per_channel, int M,
                             int K, int dtype, void* stream);

/* Replaces topsvllmSiluMulQuant as called by silu_mul_static_int8_quant
 * (csrc/src/silu_mul_static_int8_quant.cpp:11-28): x is [rows, 2d];
 * q = sat_s8(rne((silu(x[:, :d]) * x[:, d:]) * (1/scale))), the activation and the
 * reciprocal both rounded to the input dtype; scale is one value or [d]. */
int mi355q_silu_mul_static_int8_quant(int8_t* out, const void* x, const float* scale, int per_channel,
                                      long rows, int d, int dtype, void* stream);

/* The static int8 experts of FusedW8A8MoEMethod (vllm_gcu/kernels/quantization/w8a8.py:174-342) hand the
 * vendor grouped GEMM 16-bit activations together with per-expert, per-input-channel reciprocal input
 * scales [E, K] (w13_in_scales / w2_in_scales, w8a8.py:226-236; vllm_gcu/kernels/prepare_finalize.py:62-64
 * passes them through un-quantised).  Here that quantisation is a kernel of its own in front of the int8
 * grouped GEMM: for every (token, slot) id t < numel listed in the first *num_tokens_post_pad entries of
 * sorted_token_ids, with e = expert_ids[position / block_size],
 *   out[t, :] = sat_s8(rne(x[t / topk, :] * scale_rec[e, :]))   (product in fp32),
 * out is int8 [numel, K]; x and scale_rec share dtype (f16 / bf16); rows of blocks whose expert is outside
 * [0, E) are zero; max_sorted = entries of sorted_token_ids.  The vendor kernel's own rounding is not
 * part of the reference: parity with it is unpinned. */
int mi355q_moe_expert_int8_quant(int8_t* out, const void* x, const void* scale_rec,
                                 const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                 const int32_t* num_tokens_post_pad, int max_sorted, int block_size, int numel,
                                 int topk, int E, int K, int dtype, void* stream);

/* ---- MoE routing ------------------------------------------------------------
 * Replaces topsvllm's topk_softmax (csrc/src/topk_softmax.cpp:27-34):
 * softmax over E experts in fp32, top-k descending (ties to the lower index);
 * token_expert_indices[row, k] = k * M + row (may be NULL).  `renormalize`
 * divides by the row sum (done in Python by the reference's caller).  gating
 * is [M, E] of `dtype` (f16 / bf16 / f32).  E <= 1024, topk <= 64. */
int mi355q_topk_softmax(float* topk_weights, int32_t* topk_ids, int32_t* token_expert_indices,
                        const void* gating, int M, int E, int topk, int renormalize, int dtype,
                        void* stream);
/* Replaces topsvllmGroupedTopk, both overloads (csrc/src/fused_grouped_topk.cpp:22-44):
 * scores = softmax | sigmoid; with `bias` selection uses scores + bias and a
 * group's score is the sum of its two best; without it the group's max; the
 * `topk_group` best groups are kept, top-k taken among them, weights come from
 * the un-biased scores.  bias may be NULL. */
int mi355q_grouped_topk(float* topk_weights, int32_t* topk_ids, const void* gating, const float* bias,
                        int M, int E, int topk, int renormalize, int num_expert_group, int topk_group,
                        int scoring_sigmoid, int dtype, void* stream);
/* Replaces the vendor kernel behind moe_align_block_size, moe_align_block_size_pad,
 * sgl_moe_align_block_size and exts_moe_align_block_size
 * (csrc/src/moe_align_block_size.cpp:30-105, moe_align_block_size_pad.cpp:30-110,
 * exts_moe_align_block_size.cpp:16-101): stable counting sort of the flat
 * (token, slot) ids by expert, runs padded to block_size.  sorted_token_ids has
 * numel + E*(block_size-1) entries (pads = numel), expert_ids one entry per
 * block, num_tokens_post_pad one int.  valid_rows (device int32[1], optional):
 * only that many rows of topk_ids are valid.  expert_map (device int32[E],
 * optional) is applied to expert_ids. */
int mi355q_moe_align_block_size(const void* topk_ids, int ids_are_int64, int numel, int topk,
                                const int32_t* valid_rows, int num_experts, int block_size,
                                const int32_t* expert_map, int32_t* sorted_token_ids,
                                int32_t* expert_ids, int32_t* num_tokens_post_pad, void* stream);

/* ---- activation glue --------------------------------------------------------
 * silu_and_mul / silu_and_mul_pad (csrc/src/silu_and_mul.cpp:29-109,
 * silu_and_mul_pad.cpp:27-90): out[r, :d] = silu(x[r, :d]) * x[r, d:2d].
 * valid_rows (device int32[1], optional) counts leading units of rows_per_count rows each (tokens of
 * top-k slot rows): only the first *valid_rows * rows_per_count rows are processed; the product is
 * taken on the device, so a captured graph may change the count between replays. */
int mi355q_silu_and_mul(void* out, const void* x, long rows, int d, int dtype,
                        const int32_t* valid_rows, int rows_per_count, void* stream);
/* dynamic_per_token_group_fp8_quant(_with_size) and, with fuse_silu_mul,
 * silu_mul_per_token_group_quant(_with_size)
 * (csrc/src/dynamic_per_token_group_fp8_quant.cpp:15-84,
 * silu_mul_per_token_group_quant_with_size.cpp:15-89): per (row, group)
 * s = max(absmax, 1e-10) / 448, q = e4m3fn(clamp(x / s)).  x is [rows, K]
 * (or [rows, 2K] when fused); scales [rows, K / group_size] row-major. */
int mi355q_fp8_group_quant(uint8_t* out, float* scales, const void* x, long rows, int K, int group_size,
                           int fuse_silu_mul, int dtype, const int32_t* valid_rows, int rows_per_count,
                           void* stream);
/* dynamic_per_token_scaled_fp8_quant (csrc/src/dynamic_per_token_scaled_fp8_quant.cpp): one scale per row */
int mi355q_fp8_token_quant(uint8_t* out, float* scales, const void* x, int rows, int K, int dtype,
                           const int32_t* valid_rows, void* stream);
/* static_scaled_fp8_quant, silu_mul_static_fp8_quant and mul_static_fp8_quant
 * (csrc/torch_bindings.cpp:714, 291, 301; csrc/src/mul_static_fp8_quant.cpp:11-22):
 * q = e4m3fn(clamp(v / scale)) with one fp32 scale; fuse_silu_mul 0: v = x [rows, K];
 * 1: v = silu(x[:, :K]) * x[:, K:] of x [rows, 2K]; 2: v = x[:, :K] * x[:, K:] */
int mi355q_fp8_static_quant(uint8_t* out, const void* x, const float* scale, long rows, int K,
                            int fuse_silu_mul, int dtype, const int32_t* valid_rows, int rows_per_count,
                            void* stream);
/* rms_norm / fused_add_rms_norm and their fusions with the activation quantisers
 * (csrc/torch_bindings.cpp:254-272 rms_norm, fused_add_rms_norm; :277-317 *_static_fp8_quant;
 * :852-871 *_static_int8_quant; :1124-1143 *_per_token_group_quant_fp8; equivalences
 * vllm_gcu/compilation/fusion.py:104-127, 183-330).  Rows of K elements (K % 8 == 0):
 * z = x (+ residual; residual := z when given), o = act(act(z * rsqrt(mean z^2 + eps)) * weight)
 * with act() = rounding to `dtype`; quant_mode 0: out = o; 1: out = e4m3fn(o / *scale);
 * 2: out = e4m3fn per group of group_size with out_scales f32 [rows, K/group_size];
 * 3: out = int8 rne(o * act(1 / *scale)).  out may alias x when quant_mode is 0. */
int mi355q_rms_norm(void* out, float* out_scales, const void* x, void* residual, const void* weight,
                    const float* scale, float eps, long rows, int K, int quant_mode, int group_size,
                    int dtype, void* stream);
/* fp8-e4m3fn -> f16 / bf16, exact; n a multiple of 4.  Feeds fp8 activations to the int4 expert
 * GEMM of fused_moe_quant_kernel_ex (csrc/src/fused_moe_quant_kernel_ex.cpp:13-45), which the
 * reference's vendor kernel consumes directly. */
int mi355q_fp8_to_half(void* out, const uint8_t* in, long n, int out_dtype, void* stream);
/* moe_sum_pad (csrc/src/moe_sum.cpp:64-131): out[m, :] = sum_t in[m, t, :], fp32 accumulate */
int mi355q_moe_sum(void* out, const void* in, long rows, int topk, int K, int in_dtype, int out_dtype,
                   const int32_t* valid_rows, void* stream);

/* ---- fused-MoE grouped GEMM and K-contiguous skinny GEMMs -------------------
 * quant_mode: 0 = W4A16 (slab-layout int4 per expert [E, K/8, N], scales
 * [E, K/g, N], zeros per zeros_kind; g = 32, 64 or a multiple of 128), 1 = fp8-e4m3fn with 128x128 block scales
 * (w [E, N, K], a_scale f32 [Ma, K/128], w_scale f32 [E, ceil(N/128), K/128]),
 * 2 = int8 (a_scale f32 [Ma] or NULL, w_scale f32 [E, N]), 3 = unquantised
 * f16/bf16 (w [E, N, K]), 4 = W8A16 (w int8 [E, N, K], w_scale in the activation
 * dtype: [E, N] per channel with group_size <= 0 or K, [E, K/g, N] with
 * group_size g = 64 or 128, as weight_only_quant and the w8a16 experts take them,
 * csrc/src/weight_only_quant.cpp:28-101, vllm_gcu/kernels/fused_moe.py:163-169), 5 = symmetric int4 experts as in mode 0 but with fp32 group
 * scales w_scale [E, K/g, N] and a_scale = one fp32 value multiplied into every
 * output (the w4a8-fp8 experts of fused_moe_quant_kernel_ex,
 * csrc/src/fused_moe_quant_kernel_ex.cpp:13-45: a holds the fp8 activations
 * widened by mi355q_fp8_to_half, a_scale their dequantisation scale).
 *
 * mi355q_moe_gemm replaces vllmInvokeFusedMoeNonGatherQuantKernel as called by
 * fused_moe_quant_kernel / fused_moe_kernel (csrc/src/fused_moe_quant_kernel.cpp:30-200,
 * fused_moe_kernel.cpp:27-68; shapes csrc/src/native_vllm.h:236-255): for every
 * block b < num_tokens_post_pad / block_size with e = expert_ids[b] and every
 * id t < numel in the block,  out[t, :] = a[t / topk, :] @ W[e]^T  (times
 * topk_weights[t] when that pointer is given).  max_blocks = entries of
 * expert_ids.  block_size in {16, 32, 64, 128}; fp8 block-scaled, int8 and unquantised experts also 256.  For
 * those three, blocks of 256 -- and blocks of 128 from 40 rows per expert on average (numel >= 40 E) -- run the
 * MFMA tile kernels with gathered rows (prefill token counts; fp8 and unquantised: N % 128 == 0), smaller ones
 * the weight-streaming kernel.  sorted_token_ids must hold at least
 * max_blocks * block_size entries (the kernels load a block's ids before they compare the block
 * with num_tokens_post_pad).  Rows of ids that appear in no block below num_tokens_post_pad (ids
 * the alignment dropped) are not written, with or without a workspace.
 *
 * workspace (optional, may be NULL): device scratch of mi355q_moe_gemm_workspace_bytes(...) bytes for
 * the same shape.  With it, W4A16 launches whose grid would leave most of the chip idle (a long K
 * with few column tiles: the second expert GEMM of a gated MLP at prefill token counts) split K
 * into fp32 partial tiles and add them up in a second kernel; without it they run unsplit.  The
 * result differs between the two only in the order of the fp32 additions.  W4A16 with bf16
 * activations, blocks of 64 slots and two million outputs or more also stages the rows of `a` there
 * as fp16 times a power of two each (exact) for the fp16 loop; without the room the bf16 loop runs:
 * same tolerance, other bits.
 *
 * Size limits (the kernels address operands with 32-bit offsets; exceeding one is an error, not a
 * silent wrap): one expert's weights N * K elements and the activation matrix (numel / topk + 1) * K
 * elements must each stay below 2^31 elements.
 */
size_t mi355q_moe_gemm_workspace_bytes(int quant_mode, int numel, int block_size, int max_blocks, int E,
                                       int K, int N);
int mi355q_moe_gemm(void* out, const void* a, const void* w, const float* a_scale, const void* w_scale,
                    const void* w_zeros, int zeros_kind, int quant_mode, int group_size,
                    const float* topk_weights, const int32_t* sorted_token_ids, const int32_t* expert_ids,
                    const int32_t* num_tokens_post_pad, int numel, int topk, int block_size,
                    int max_blocks, int E, int K, int N, int act_dtype, int out_dtype, int w_layout,
                    void* workspace, size_t workspace_bytes, void* stream);
/* Dense calls of the same kernels (quant_mode 1..4), replacing topsatenLinearQuant
 * as called by linear_quant (csrc/src/linear_quant.cpp:16-95, fp8 block-scaled
 * C = sum_kb (A_kb B_kb^T) As Bs) and by weight_only_quant
 * (csrc/src/weight_only_quant.cpp:28-101, W8A16).  w is [N, K]; bias [N] in
 * the output dtype or NULL.  N * K and M * K must each stay below 2^31 elements. */
int mi355q_kcontig_gemm(void* out, const void* a, const void* w, const float* a_scale,
                        const void* w_scale, const void* bias, int quant_mode, int group_size, int M,
                        int K, int N, int act_dtype, int out_dtype, int w_layout, void* stream);
/* Weight layout of quant_mode 1..4 (w_layout above).  0: row-major [E, N, K], the checkpoint's
 * and the reference's (vllm_gcu/kernels/quantization/fp8.py:72-166 keeps it).  1: "kslab",
 * this library's streaming order of the same bytes, N % 64 == 0:
 * [E][N/64][K/128][4 tiles of 16 rows][2*elem_bytes vectors][64 lanes][16 B], where lane l of
 * vector v of tile i holds bytes (128 kb + 32 (l/16)) * elem_bytes + 16 v .. +16 of row
 * 64 ng + 16 i + l%16 -- each wavefront load reads one contiguous KiB.  No counterpart in
 * the reference (load-time conversion, like its int4 rearrange). */
int mi355q_kslab_repack(const void* src, void* dst, int batch, int N, int K, int elem_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355Q_H */

/*
 * taac_hip.h - C ABI of libtaac_hip.so: the gfx950 (MI355X) kernel path of the TAAC-2026 unified
 * pCVR token backbone.
 *
 * Conventions shared by every entry point
 *   - All data pointers are DEVICE pointers owned by the caller; nothing is allocated or freed here.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream). Work is enqueued
 *     asynchronously on it; the call returns as soon as the launches are queued.
 *   - Return value: TAAC_OK (0) or a negative TAAC_ERR_* code. After a failure taac_last_error()
 *     returns a human-readable message (thread-local storage, valid until the next call on that thread).
 *   - Arguments are validated on the host before any kernel is launched; a rejected call launches nothing.
 *   - `dtype` is a taac_dtype value.
 *   - No global mutable state besides the thread-local error string (and the scratch array of
 *     taac_rmsnorm_bwd_static): calls from different host threads and on different streams are independent.
 *     Behaviour is chosen by arguments only; no environment variable is read. taac_test_hooks (last declaration) sets
 *     two process-wide test switches that change no result.
 *
 * Each declaration cites the reference interface it replaces (path:line under the reference tree,
 * Puiching-Memory/TAAC_2026). The reference has no C ABI on this path: its operators are Python
 * functions that dispatch to torch / Triton / TileLang; the entry points here are what a
 * `register_*_kernel` hook or a drop-in Python operator binds with ctypes.
 */
#ifndef TAAC_HIP_H
#define TAAC_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TAAC_ABI_VERSION 9

enum taac_status {
  TAAC_OK = 0,
  TAAC_ERR_INVALID_VALUE = -1, /* bad shape / size / enum: the Python layer raises ValueError */
  TAAC_ERR_UNSUPPORTED = -2,   /* valid request outside the kernels' envelope: RuntimeError   */
  TAAC_ERR_LAUNCH = -3         /* HIP reported an error at launch: RuntimeError                */
};

enum taac_dtype { TAAC_F32 = 0, TAAC_BF16 = 1, TAAC_F16 = 2 };

/* Epilogues of the dense-layer entry points (taac_linear_*). */
enum taac_epilogue {
  TAAC_EPI_NONE = 0,   /* out = a @ w^T (+ bias)                                              */
  TAAC_EPI_RESIDUAL = 1, /* out = residual + a @ w^T (+ bias); out may alias residual          */
  TAAC_EPI_SWIGLU = 2  /* w is [2F, K]; out[M, F] = silu(g) * u (gate_first) or g * silu(u)    */
};

/* Bits of the `is_causal` argument of the key-length attention entry points (forward, scaled, training pair). */
#define TAAC_ATTN_CAUSAL 1           /* key j is visible to query i only if j <= i                                */
#define TAAC_ATTN_REGISTER_STAGING 2 /* stage K / V chunks through registers instead of direct global -> LDS       */
                                     /* transfers: same arithmetic and results, kept as a comparison route        */

/* Bits of the `flags` argument of taac_backbone_fwd. */
#define TAAC_BACKBONE_DENSE_TOKENS 1  /* run the dense layers over the padded positions too                        */
#define TAAC_BACKBONE_SPLIT_OUT_FFN 2 /* out projection and feed-forward half as two kernels instead of one        */
#define TAAC_BACKBONE_FP8 4           /* the four dense layers of a block with e4m3 MFMA operands and per-tensor   */
                                      /* scales (amax / 448); D = 256, F a multiple of 64, plain attention layer   */
#define TAAC_BACKBONE_ROW_MAJOR_QKV 8 /* keep q | k | v and the attention output of the workspace as [M, 3D] / [M, D] */
                                      /* rows instead of per-head planes (comparison route; same results)          */

int taac_abi_version(void);
const char* taac_last_error(void);

/* TEST-ONLY, not part of the drop-in surface (no counterpart in the reference): process-wide switches for the test
 * suite that change scheduling and never a result. max_workgroups > 0 caps the grid of the persistent dense kernels
 * (taac_norm_linear*_fwd, taac_linear_fp8, taac_norm_linear_fp8_fwd) and the number of units the fused feed-forward
 * kernels spread their last round over, so that small test inputs walk several token tiles per workgroup; 0 removes
 * the cap. fp8_tiled != 0 routes taac_linear_fp8 to its generic tiled kernel for every shape. Both start at 0. */
void taac_test_hooks(int32_t max_workgroups, int32_t fp8_tiled);

/*
 * RMSNorm forward: y[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w, fp32 accumulation, one rounding
 * to the storage dtype. x, y: [rows, cols] contiguous; w: [cols] in the same dtype as x.
 * Replaces: rms_norm / _torch_rms_norm (src/taac2026/infrastructure/accelerators/normalization/rms_norm.py:377-401,
 * 71-73) and the Triton forward kernel (normalization/kernels/triton.py:30-50). Matches the signature
 * a kernel registered through register_rms_norm_kernel receives (rms_norm.py:31,66-68).
 */
int taac_rmsnorm_fwd(const void* x, const void* w, void* y, int64_t rows, int32_t cols, float eps, int dtype,
                     void* stream);

/*
 * LayerNorm forward: y = (x - mean) * rsqrt(var + eps) * w + b, biased variance computed from centred
 * values, fp32 accumulation. Shapes as taac_rmsnorm_fwd, b: [cols].
 * Replaces: layer_norm / _torch_layer_norm (normalization/layer_norm.py:261-280, 65-66) and the Triton
 * inference kernel (normalization/kernels/triton.py:224-247); hook signature of register_layer_norm_kernel
 * (layer_norm.py:24,60-62).
 */
int taac_layernorm_fwd(const void* x, const void* w, const void* b, void* y, int64_t rows, int32_t cols, float eps,
                       int dtype, void* stream);

/*
 * Backward of taac_rmsnorm_fwd / taac_layernorm_fwd. With g = dy * w and x_hat the normalised row:
 *   RMSNorm:   dx = rstd * (g - x_hat * mean(g * x_hat));            dw = sum over rows of dy * x_hat
 *   LayerNorm: dx = rstd * (g - mean(g) - x_hat * mean(g * x_hat));  dw as above; db = sum over rows of dy
 * The row statistics are recomputed from x (nothing is saved by the forward). x, dy, dx: [rows, cols] contiguous;
 * w, dw, db: [cols]; all in `dtype`, fp32 arithmetic. dw / db may be NULL (not wanted). workspace: device memory for
 * taac_norm_bwd_workspace_floats(rows, cols, layer_norm) floats (per-workgroup partial sums of dw / db, added in a
 * fixed order: the result does not depend on scheduling). Rows of whole 16-byte vectors (8 elements, 4 for fp32), at
 * most 256 of them, with 16-byte aligned tensors take the one-pass vector kernel; every other shape takes a generic
 * kernel (one workgroup per row at a time, the row swept four times).
 * Replaces: the Triton / TileLang backward kernels and their host-side partial sums
 * (accelerators/normalization/kernels/triton.py:82-116, 276-320; rms_norm.py:294-340, layer_norm.py:170-258).
 */
int64_t taac_norm_bwd_workspace_floats(int64_t rows, int32_t cols, int layer_norm);
int taac_rmsnorm_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, float* workspace,
                     int64_t workspace_floats, int64_t rows, int32_t cols, float eps, int dtype, void* stream);
int taac_layernorm_bwd(const void* x, const void* w, const void* dy, void* dx, void* dw, void* db, float* workspace,
                       int64_t workspace_floats, int64_t rows, int32_t cols, float eps, int dtype, void* stream);

/*
 * taac_rmsnorm_bwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the per-workgroup partial sums of dw live in a device array that is part of the
 * library image (TAAC_RMSNORM_BWD_STATIC_MAX_COLS * 1024 floats = 8 MiB per GPU, held until the process ends) instead
 * of a caller workspace. No counterpart in the reference. Arguments and results as taac_rmsnorm_bwd (bit-identical);
 * cols above TAAC_RMSNORM_BWD_STATIC_MAX_COLS are rejected with TAAC_ERR_UNSUPPORTED. The call allocates and frees
 * nothing. All calls on one GPU share the array: calls that overlap on one GPU (different streams or host threads)
 * race on it and must be serialised by the caller; calls on one stream are ordered and safe.
 * The array's device address is looked up (hipGetSymbolAddress) by the first call on each GPU: make one ordinary call
 * per GPU (rows = 0 is enough) before the first call under stream capture, so that the lookup, which may load the code
 * object, does not happen inside a capture.
 */
#define TAAC_RMSNORM_BWD_STATIC_MAX_COLS 2048
int taac_rmsnorm_bwd_static(const void* x, const void* w, const void* dy, void* dx, void* dw, int64_t rows,
                            int32_t cols, float eps, int dtype, void* stream);

/*
 * Key-padding-masked attention forward: o = softmax(q k^T / sqrt(d) + mask) v per (batch, head), softmax in
 * fp32, bf16/fp16 MFMA operands. Key j of batch b is visible iff j < key_lengths[b] (and j <= query index when
 * is_causal has TAAC_ATTN_CAUSAL set; is_causal is a bit set, 0 / 1 keep their plain meaning).
 * key_lengths == NULL means every key is visible. Rows with no visible key produce zeros.
 * q/o: logical shape (B, H, Tq, d); k/v: (B, H, Tk, d). *_strides are ELEMENT strides of the four logical
 * dimensions, so (B,H,T,d)-contiguous and (B,T,H,d)-contiguous tensors are both read in place; the last
 * stride must be 1, the others multiples of 8, and base pointers 16-byte aligned. d must be a multiple of 8, <= 128.
 * zero_padded_queries != 0 (requires Tq == Tk): query rows t >= key_lengths[b] are not read and not computed; they are
 * written as zeros (1) or left untouched (2).
 * dtype: TAAC_BF16 or TAAC_F16.
 * Replaces: flash_attention's kernel call `_flash_attention_kernel(q, k, v, key_lengths)`
 * (accelerators/attention/flash_attention.py:338-367, hook at :26,102-104) and the TileLang inference kernel
 * (accelerators/attention/kernels/tilelang.py:36-138); the strided form also replaces the four layout copies of
 * scaled_dot_product_attention (infrastructure/modeling/sequence.py:81-116).
 */
int taac_flash_attn_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths, void* o, int32_t B,
                        int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                        const int64_t k_strides[4], const int64_t v_strides[4], const int64_t o_strides[4],
                        int is_causal, int zero_padded_queries, int dtype, void* stream);

/*
 * taac_flash_attn_fwd with one positive factor per query row and per key row, shared by the heads, and one factor
 * per query feature:
 *   scores = (q_row_scale[b, i] * q[b, h, i, :] * q_col_scale[h, :]) . (k_row_scale[b, j] * k[b, h, j, :]) / sqrt(d).
 * q_row_scale: fp32 [B, Tq] contiguous or NULL (all ones); k_row_scale: fp32 [B, Tk] or NULL; q_col_scale: fp32 [H, d],
 * 16-byte aligned, or NULL. The query row factor joins the softmax scale (no rounding); the query features and the key rows are
 * multiplied in fp32 and rounded once to the storage dtype on their way to the MFMA. Factors of rows in the padding
 * are not read. Everything else as taac_flash_attn_fwd. (The weights of a query norm and of a key norm act on a score
 * only through their product, so q_col_scale = query weight * key weight applies both without touching the keys.)
 * Use: a per-token normalisation statistic that is only known after the projection that produced q and k has
 * finished (RMSNorm over the model width: the factor is rsqrt(mean(x^2) + eps), taac_norm_linear_qk_fwd +
 * taac_row_rstd), so that the normalisation costs no pass over q and k. Replaces, together with those, query_norm /
 * key_norm of UnifiedSelfAttention.forward (experiments/symbiosis/backbone.py:33-36).
 */
int taac_flash_attn_scaled_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                               const float* q_row_scale, const float* k_row_scale, const float* q_col_scale, void* o,
                               int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                               const int64_t k_strides[4], const int64_t v_strides[4], const int64_t o_strides[4],
                               int is_causal, int zero_padded_queries, int dtype, void* stream);

/*
 * taac_flash_attn_scaled_fwd that also reduces max |o| over everything it writes into *amax_out (device float, cleared
 * by the call): the per-tensor FP8 scale of the output projection that consumes o, taken in the kernel's epilogue
 * instead of in a pass of its own. Padded query rows that are not written (zero_padded_queries = 2) do not count.
 * No counterpart in the reference (it has no FP8 code).
 */
int taac_flash_attn_amax_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                             const float* q_row_scale, const float* k_row_scale, const float* q_col_scale, void* o,
                             float* amax_out, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                             const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                             const int64_t o_strides[4], int is_causal, int zero_padded_queries, int dtype, void* stream);

/*
 * Attention under a structured mask: key j is visible to query i of sample b iff
 *   structural[i, j] AND key_valid[b, j]      (AND j < key_lengths[b] when key_lengths is given),
 * with structural shared by the batch and the heads. That is the form of the reference's model-level masks:
 * TokenFormer's per-layer full / sliding-window mask with always-visible separator keys and an all-seeing target query
 * (_bfts_attention_mask, experiments/tokenformer/model.py:474-503) and Symbiosis' role-metadata mask
 * (MetadataAttentionMask.forward, experiments/symbiosis/attention.py:21-60), both ANDed with the key padding; the
 * reference's accelerated attention path rejects them (flash_attention.py:183-209) and falls back to torch SDPA.
 * struct_bits: uint32 [Tq, ceil(Tk / 32)], bit j % 32 of word j / 32 of row i = structural[i, j], bits beyond Tk zero
 * (taac_mask_pack_bits); block_any: uint8 [ceil(Tq / 128), ceil(Tk / 64)] from taac_mask_block_any: 64-key chunks that
 * no query of a 128-row block can see are neither loaded nor computed, 32-key tiles that no query of a wavefront sees
 * are skipped, fully visible tiles skip the bit tests. valid_bits: uint32 [B, ceil(Tk / 32)] or NULL (all valid).
 * self_bits: uint32 [B, ceil(Tq / 32)] or NULL; a flagged query row returns its own value row (the reference's
 * fallback for padded queries, which attend to themselves only; requires Tq == Tk). Rows with no visible key give
 * zeros. The row / feature factors are those of taac_flash_attn_scaled_fwd (NULL: none). Everything else as
 * taac_flash_attn_fwd; no is_causal (put the triangle into structural); Tk <= 4096.
 * struct_sample_stride: 0 for one structural matrix shared by the batch, else the number of 32-bit words between the
 * matrices of consecutive samples (at least Tq * ceil(Tk / 32)): per-sample structure, as taac_mask_front_bits writes
 * it for samples whose valid tokens were moved to the front; block_any may then be NULL (no chunk is skipped on
 * structure).
 */
int taac_flash_attn_masked_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                               const uint32_t* struct_bits, int64_t struct_sample_stride, const uint8_t* block_any,
                               const uint32_t* valid_bits,
                               const uint32_t* self_bits, const float* q_row_scale, const float* k_row_scale,
                               const float* q_col_scale, void* o, int32_t B, int32_t H, int32_t Tq, int32_t Tk,
                               int32_t d, const int64_t q_strides[4], const int64_t k_strides[4],
                               const int64_t v_strides[4], const int64_t o_strides[4], int zero_padded_queries,
                               int dtype, void* stream);

/*
 * taac_flash_attn_masked_fwd (same mask, same result up to the summation order of the softmax) for masks in which a
 * 32-query tile sees only a few key columns: sliding windows with a few always-visible key columns and query rows, the
 * upper layers of TokenFormer's mask (experiments/tokenformer/model.py:474-503). The structure arrives in compact form
 * (taac_mask_compact): per 32-query tile the ascending list of key columns some query of the tile can see, cut into
 * compact tiles of 32 keys, and per query row one word per compact tile. One wavefront per 32-query tile works on its
 * own: it visits the compact tiles that can hold a valid key of the sample (valid_bits, key_lengths), gathers their K
 * rows straight from global memory into MFMA fragments and their V rows through a wavefront-private LDS tile, and
 * applies the row's word. A tile whose query rows are all self-only or in the padding visits nothing. The time follows
 * the number of visible key columns per query tile (in units of 32) instead of the number of 64-key chunks a 128-query
 * block touches; for dense masks the chunked kernel is faster, so the caller chooses.
 * compact_bits: uint32 [samples, Tq, ceil(Tk / 32)]; compact_keys: int32 [samples, ceil(Tq / 32), 32 ceil(Tk / 32)];
 * compact_tiles: uint64 [samples, ceil(Tq / 32), 64]; samples = 1 (compact_sample_stride = 0) for a structure shared by
 * the batch, else B with compact_sample_stride = Tq * ceil(Tk / 32).
 * Head dims 32 and 64, Tk <= 2048, key / value row strides that fit 32-bit byte offsets; anything else is
 * TAAC_ERR_UNSUPPORTED (use taac_flash_attn_masked_fwd). Other arguments as taac_flash_attn_masked_fwd.
 */
int taac_flash_attn_sparse_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                               const uint32_t* compact_bits, int64_t compact_sample_stride, const int32_t* compact_keys,
                               const uint64_t* compact_tiles, const uint32_t* valid_bits, const uint32_t* self_bits,
                               const float* q_row_scale, const float* k_row_scale, const float* q_col_scale, void* o,
                               int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                               const int64_t k_strides[4], const int64_t v_strides[4], const int64_t o_strides[4],
                               int zero_padded_queries, int dtype, void* stream);

/*
 * Compact form of a structure matrix for taac_flash_attn_sparse_fwd. For sample s and query tile t (rows 32 t .. 32 t + 31
 * below Tq): compact_keys[s, t, :] = the key columns j with struct_bits[row, j] set for some row of the tile, ascending,
 * then -1; compact_tiles[s, t, c] = bit w set iff compact tile c (keys 32 c .. 32 c + 31 of that list) holds a key of
 * word w (keys 32 w .. 32 w + 31 of Tk), 0 for tiles beyond the list; compact_bits[s, row, c] = bit j set iff the row
 * sees key compact_keys[s, row / 32, 32 c + j]. samples = 1 for a structure shared by the batch, else B with
 * struct_sample_stride words between the samples' matrices. Tk <= 2048.
 * No counterpart in the reference (its fallback passes a dense bool mask to torch SDPA).
 */
int taac_mask_compact(const uint32_t* struct_bits, int32_t samples, int32_t Tq, int32_t Tk, int64_t struct_sample_stride,
                      uint32_t* compact_bits, int32_t* compact_keys, uint64_t* compact_tiles, void* stream);

/* Packs a row-major bool matrix (one byte per element, nonzero = true) [rows, cols] into bit rows
 * [rows, ceil(cols / 32)]: the struct_bits / valid_bits / self_bits of taac_flash_attn_masked_fwd. */
int taac_mask_pack_bits(const void* mask, int64_t rows, int32_t cols, uint32_t* bits, void* stream);

/* block_any [ceil(Tq / 128), ceil(Tk / 64)] of struct_bits [Tq, ceil(Tk / 32)] for taac_flash_attn_masked_fwd. */
int taac_mask_block_any(const uint32_t* struct_bits, int32_t Tq, int32_t Tk, uint8_t* block_any, void* stream);

/*
 * Training pair of taac_flash_attn_fwd (key-length mask, optional causal triangle; head_dim <= 64 for the backward).
 * taac_flash_attn_train_fwd additionally writes lse: fp32 [B, H, Tq] contiguous, the natural-log sum of exp of the
 * scaled scores of every query row (-inf for rows without a visible key and for padded rows).
 * taac_flash_attn_bwd: with P = exp(q k^T / sqrt(d) - lse) on the visible pairs and D_i = sum_d o[i, d] dout[i, d],
 *   dv = P^T dout,  dS = P * (dout v^T - D) / sqrt(d),  dq = dS k,  dk = dS^T q
 * for the same mask arguments as the forward. o is the forward's output, dout its gradient (logical (B, H, Tq, d) like
 * q, own strides); dq / dk / dv have the logical shapes of q / k / v and their own element strides (same rules as the
 * forward). delta: workspace, fp32 [B, H, Tq]. With zero_padded_queries the padded query rows carry no gradient (dq
 * rows are zero); gradients of keys at or beyond key_lengths[b] are zero. Every output element has one writer and a
 * fixed summation order (two kernels, each recomputing the scores), so results are reproducible run to run.
 * Replaces: the TileLang training forward (accelerators/attention/kernels/tilelang.py:287-390) and backward
 * preprocess + backward kernels (:405-435, 598-699), which accumulate dq with floating-point atomics.
 */
int taac_flash_attn_train_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths, void* o,
                              float* lse, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                              const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                              const int64_t o_strides[4], int is_causal, int zero_padded_queries, int dtype,
                              void* stream);
int taac_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                        const int32_t* key_lengths, void* dq, void* dk, void* dv, float* delta, int32_t B, int32_t H,
                        int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4], const int64_t k_strides[4],
                        const int64_t v_strides[4], const int64_t o_strides[4], const int64_t do_strides[4],
                        const int64_t dq_strides[4], const int64_t dk_strides[4], const int64_t dv_strides[4],
                        int is_causal, int zero_padded_queries, int dtype, void* stream);

/*
 * Training pair for attention under a mask that is not a key prefix or a causal triangle.
 * taac_flash_attn_masked_train_fwd: taac_flash_attn_masked_fwd (structured mask, no row / feature factors) that also
 * writes lse as taac_flash_attn_train_fwd does (-inf for rows without a visible key; the value written for a flagged
 * self row is not used by the backward). dropout_mask (NULL: none): the keep mask [B, H, Tq, Tk] and scale 1 / (1 - p) of
 * taac_flash_attn_train_dropout_fwd, applied behind the normaliser over the visible keys; not with self_bits.
 * taac_flash_attn_mask_bwd: taac_flash_attn_bwd with the visible pairs given as bytes: visible[b * visible_batch_stride +
 * h * visible_head_stride + i * Tk + j] != 0 iff key j is visible to query i (strides in elements, 0 = shared by the
 * batch / the heads; AND j < key_lengths[b] when key_lengths is given; AND key_valid[b * Tk + j] != 0 when key_valid is
 * given - the factored form structure[i, j] & key_valid[b, j] then needs one shared matrix and B * Tk bytes instead of B
 * matrices). An invisible pair has probability 0 in dV and dS. A query row whose lse is +inf contributes nothing and
 * receives a zero gradient (how a caller takes rows out: the self-only rows of a structured mask).
 * Any bool mask the forward applied can be written out this way; rows of flagged self queries are written as all
 * invisible, and the caller adds dout of those rows to dv (o = v there).
 * Replaces: what torch autograd derives for F.scaled_dot_product_attention under the bool masks of the reference's models
 * (experiments/symbiosis/attention.py:21-60, experiments/tokenformer/model.py:474-503, flash_attention.py:183-209), which
 * its accelerated path rejects.
 */
int taac_flash_attn_masked_train_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                     const uint32_t* struct_bits, int64_t struct_sample_stride, const uint8_t* block_any,
                                     const uint32_t* valid_bits, const uint32_t* self_bits, const uint8_t* dropout_mask,
                                     float dropout_scale, void* o, float* lse, int32_t B,
                                     int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                                     const int64_t k_strides[4], const int64_t v_strides[4], const int64_t o_strides[4],
                                     int zero_padded_queries, int dtype, void* stream);
int taac_flash_attn_mask_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                             const int32_t* key_lengths, const uint8_t* visible, int64_t visible_batch_stride,
                             int64_t visible_head_stride, const uint8_t* key_valid, void* dq, void* dk, void* dv,
                             float* delta, int32_t B, int32_t H,
                             int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4], const int64_t k_strides[4],
                             const int64_t v_strides[4], const int64_t o_strides[4], const int64_t do_strides[4],
                             const int64_t dq_strides[4], const int64_t dk_strides[4], const int64_t dv_strides[4],
                             int zero_padded_queries, int dtype, void* stream);

/*
 * Training forward and backward with dropout on the attention probabilities, the mask supplied by the caller:
 * dropout_mask is uint8 [B, H, Tq, Tk] contiguous (non-zero = keep), dropout_scale = 1 / (1 - p) >= 1. The softmax
 * normaliser and lse are those of the undropped probabilities; out = ((keep ? P * dropout_scale : 0) V); the backward
 * forms dV from the dropped probabilities and dS = P * ((keep ? dP * dropout_scale : 0) - D) / sqrt(d) with
 * D = rowsum(dO * out). Every other argument as in taac_flash_attn_train_fwd / taac_flash_attn_bwd (key-length and
 * causal masks; the backward for head dims up to 64).
 * Replaces: flash_attention_training_forward_kernel / flash_attention_backward_kernel with use_dropout
 * (infrastructure/accelerators/attention/kernels/tilelang.py:165-283, 463-597); the mask is the one
 * _build_tilelang_dropout_mask draws (attention/flash_attention.py:316-325).
 */
int taac_flash_attn_train_dropout_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                      const uint8_t* dropout_mask, float dropout_scale, void* o, float* lse, int32_t B,
                                      int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                                      const int64_t k_strides[4], const int64_t v_strides[4], const int64_t o_strides[4],
                                      int is_causal, int zero_padded_queries, int dtype, void* stream);
int taac_flash_attn_dropout_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout,
                                const float* lse, const int32_t* key_lengths, const uint8_t* dropout_mask,
                                float dropout_scale, void* dq, void* dk, void* dv, float* delta, int32_t B, int32_t H,
                                int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4], const int64_t k_strides[4],
                                const int64_t v_strides[4], const int64_t o_strides[4], const int64_t do_strides[4],
                                const int64_t dq_strides[4], const int64_t dk_strides[4], const int64_t dv_strides[4],
                                int is_causal, int zero_padded_queries, int dtype, void* stream);

/*
 * Dense layer, bf16 storage / bf16 MFMA / fp32 accumulation: out = epilogue(a @ w^T + bias).
 * a: [M, K] with row stride lda (elements); w: [N, K] contiguous (torch nn.Linear layout, [out, in]);
 * bias: [N] bf16 or NULL; residual: [M, N_out] with row stride ldo or NULL; out: [M, N_out] with row stride ldo,
 * where N_out = N, or N / 2 for TAAC_EPI_SWIGLU. K must be a multiple of 8, lda/ldo multiples of 8.
 * TAAC_EPI_SWIGLU: rows [0, N/2) of w produce g, rows [N/2, N) produce u (torch .chunk(2, -1) order);
 * gate_first != 0 gives silu(g) * u (experiments/symbiosis/backbone.py:19-21), gate_first == 0 gives g * silu(u)
 * (experiments/baseline/model.py:108-113).
 * Replaces: the nn.Linear calls of UnifiedSelfAttention / SwiGLUFeedForward (experiments/symbiosis/backbone.py:
 * 11-47) together with the elementwise SiLU-gate and the residual adds of UnifiedInteractionBlock (:58-68).
 */
int taac_linear_bf16(const void* a, int64_t lda, const void* w, const void* bias, const void* residual, void* out,
                     int64_t ldo, int64_t M, int32_t N, int32_t K, int epilogue, int gate_first, void* stream);

/*
 * taac_linear_bf16 with float16 operands, bias, residual and output (fp32 accumulation, v_mfma_f32_32x32x16_f16): the
 * dense layers of a model that runs in float16, the 16-bit type of the reference's GPU tests
 * (tests/gpu/infrastructure/accelerators/test_tilelang_ops_cuda.py:61-73). Same arguments, epilogues and alignment rules.
 * Replaces: nn.Linear / F.linear on float16 tensors (experiments/symbiosis/backbone.py:14-21, 29, 32).
 */
int taac_linear_f16(const void* a, int64_t lda, const void* w, const void* bias, const void* residual, void* out,
                    int64_t ldo, int64_t M, int32_t N, int32_t K, int epilogue, int gate_first, void* stream);

/*
 * Backward pieces of a dense layer y = a w^T + b that are not themselves a forward-shaped product (the input gradient
 * dy w is one: taac_linear_bf16 with the transposed weight):
 *   taac_linear_wgrad: dw[n, k] = sum_m dy[m, n] * a[m, k] and (db != NULL) db[n] = sum_m dy[m, n].
 *     dy: [M, N] bf16 (row stride ldy), a: [M, K] bf16 (row stride lda), dw: [N, K], db: [N], both of out_dtype
 *     (TAAC_BF16 or TAAC_F32), contiguous. fp32 accumulation; the token range is split over workgroups and the splits
 *     are added in a fixed order (bit-reproducible). workspace: taac_linear_wgrad_workspace_floats(M, N, K) floats.
 *   taac_swiglu_bwd: gu: [M, 2F] pre-activations (g | u); hidden (or NULL) = silu(g) * u (gate_first) or g * silu(u);
 *     with dhidden [M, F]: dgu (or NULL) = (dg | du), dg = dhidden * u * silu'(g), du = dhidden * silu(g) (roles swapped
 *     without gate_first). bf16, fp32 arithmetic, one rounding per output.
 * Replaces: what torch autograd derives for nn.Linear and F.silu(gate) * value in the reference's training runs
 * (experiments/symbiosis/backbone.py:11-21, 24-48).
 */
int64_t taac_linear_wgrad_workspace_floats(int64_t M, int32_t N, int32_t K);
int taac_linear_wgrad(const void* dy, int64_t ldy, const void* a, int64_t lda, void* dw, void* db, float* workspace,
                      int64_t workspace_floats, int64_t M, int32_t N, int32_t K, int out_dtype, void* stream);
int taac_swiglu_bwd(const void* gu, int64_t ldgu, const void* dhidden, int64_t lddh, void* dgu, int64_t lddgu, void* hidden,
                    int64_t ldh, int64_t M, int32_t F, int gate_first, void* stream);

/*
 * The activation part of the feed-forward backward in one kernel (model width D = 128 / 256, F a multiple of 32):
 *   pre = h w_up^T + b_up, dhidden = dy w_down               -- recomputed in fp32 registers, never written --
 *   hidden [M, F] = act(pre), grad_pre [M, 2F] = d act / d pre * dhidden      (formulas of taac_swiglu_bwd)
 * h: [M, D] input of the up projection (the normalised rows), dy: [M, D] gradient of the feed-forward output; both bf16.
 * packed: the blob written by taac_swiglu_ffn_bwd_pack_weights for (w_up [2F, D], w_down [D, F]),
 * taac_swiglu_ffn_bwd_packed_bytes(D, F) bytes (-1: shape not covered). b_up: [2F] or NULL.
 * The outputs are the operands of the two weight gradients (taac_linear_wgrad) and of the input gradient
 * grad_pre w_up. Replaces: the up projection, dy w_down and the activation backward that torch autograd runs as
 * separate kernels for SwiGLUFeedForward (experiments/symbiosis/backbone.py:11-21).
 */
int64_t taac_swiglu_ffn_bwd_packed_bytes(int32_t D, int32_t F);
int taac_swiglu_ffn_bwd_pack_weights(const void* w_up, const void* w_down, void* packed, int32_t D, int32_t F, void* stream);
int taac_swiglu_ffn_bwd_hidden(const void* h, int64_t ldh, const void* dy, int64_t lddy, const void* packed,
                               const void* b_up, void* hidden, int64_t ldhid, void* grad_pre, int64_t ldgp, int64_t M,
                               int32_t D, int32_t F, int gate_first, void* stream);

/*
 * Fused feed-forward half of a block, one kernel:
 *   out = residual + down( silu(g) * u ),   g, u = chunk2( up( norm_weight ? rmsnorm(x, norm_weight, eps) : x ) )
 * x: [M, D] bf16 (row stride ldx); w_up: [2F, D]; b_up: [2F] or NULL; w_down: [D, F]; b_down: [D] or NULL;
 * residual: [M, D] (row stride ldr) or NULL; out: [M, D] (row stride ldo), may alias residual and x.
 * packed_weights: NULL, or the blob written by taac_ffn_pack_weights for the same (w_up, w_down); when given,
 * w_up / w_down are not read (they may be NULL) and weight staging reads contiguous memory.
 * D must be 128 or 256, F a multiple of 32. The [M, 2F] projection and the [M, F] gated hidden state are never
 * written to memory. gate_first as in taac_linear_bf16.
 * rows / n_rows: both NULL (every row 0..M-1 is a token), or a row index as written by taac_valid_rows: the tokens are
 * rows[0 .. *n_rows) of x / residual / out (*n_rows <= M, read on the device), all other rows are neither read nor
 * written - this is how the layers skip the padded positions of a padded [B, T, D] batch.
 * norm_folded: 0, or what the packed blob already holds - TAAC_FOLDED_NORM (needs norm_weight and packed_weights; 1, as
 * before the second flag existed): the blob is that of taac_ffn_pack_weights_norm / _folded, i.e. the norm's weight is
 * already part of the up projection, and the kernel multiplies the rows by rsqrt(mean(x^2) + eps) only;
 * TAAC_FOLDED_ACTIVATION (taac_swiglu_ffn_fwd, taac_attn_out_ffn_fwd and taac_attn_out_ffn_heads_fwd on packed weights):
 * the blob is that of taac_ffn_pack_weights_folded with fold_activation, whose up projection carries the constants of
 * silu(g) * u (see there).
 * Replaces: ffn_norm + SwiGLUFeedForward.forward + residual add of UnifiedInteractionBlock.forward
 * (experiments/symbiosis/backbone.py:19-21, 66-67).
 */
int taac_swiglu_ffn_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w_up,
                        const void* b_up, const void* w_down, const void* b_down, const void* packed_weights,
                        const void* residual, int64_t ldr, void* out, int64_t ldo, int64_t M, int32_t D, int32_t F,
                        int gate_first, const int32_t* rows, const int32_t* n_rows, int norm_folded, void* stream);

/*
 * Plain SiLU feed-forward (OneTrans' FeedForward), one kernel with the hidden state in registers:
 *   out = residual + fc2( silu( fc1( norm_weight ? rmsnorm(x, norm_weight, eps) : x ) ) )
 * fc1: [F, D] with bias b1 [F] or NULL, fc2: [D, F] with bias b2 [D] or NULL, both handed over as the blob written by
 * taac_silu_mlp_pack_weights (taac_silu_mlp_packed_bytes bytes; -1: unsupported shape). x, residual (or NULL), out,
 * row strides, rows / n_rows as in taac_swiglu_ffn_fwd. D must be 128 or 256, F a multiple of 32.
 * Replaces: FeedForward.forward in eval mode (experiments/onetrans/model.py:33-44: Linear -> SiLU -> Dropout ->
 * Linear), with the ffn_norm and the residual add of OneTransBlock.forward (:107) when they are passed.
 */
int64_t taac_silu_mlp_packed_bytes(int32_t D, int32_t F);
int taac_silu_mlp_pack_weights(const void* w1, const void* w2, void* packed, int32_t D, int32_t F, void* stream);
int taac_silu_mlp_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* b1, const void* b2,
                      const void* packed_weights, const void* residual, int64_t ldr, void* out, int64_t ldo, int64_t M,
                      int32_t D, int32_t F, const int32_t* rows, const int32_t* n_rows, void* stream);

/*
 * Attention output projection + residual and the feed-forward half of a block in one kernel:
 *   x1  = residual + (attn @ w_out^T + out_bias)
 *   out = x1 + down( silu(g) * u ) + b_down,   g, u = chunk2( up( norm_weight ? rmsnorm(x1, norm_weight, eps) : x1 ) )
 * attn: [M, D] bf16 attention output (row stride ld_attn); residual: [M, D] block input (row stride ldr, required);
 * out: [M, D] (row stride ldo), may alias residual, not attn. packed_out_weights: blob of taac_linear_pack_weights for
 * the [D, D] projection; packed_ffn_weights: blob of taac_ffn_pack_weights with gate_first = 1 (both required);
 * out_bias / b_up / b_down may be NULL. x1 is rounded to bf16 as the reference's residual stream is, but is never
 * written to memory: it stays in the accumulators of the down projection, so the final sum x1 + down + b_down is
 * rounded once (the two-kernel route rounds down + b_down first). D must be 128 or 256, F a multiple of 32.
 * rows / n_rows, norm_folded: as in taac_swiglu_ffn_fwd (rows of residual and out). attn_rows: NULL, or (with rows) the
 * row of attn that holds token i when attn is laid out differently (taac_front_rows).
 * Replaces: attention.out + residual add and ffn_norm + SwiGLUFeedForward.forward + residual add of
 * UnifiedInteractionBlock.forward (experiments/symbiosis/backbone.py:47, 64-67).
 */
int taac_attn_out_ffn_fwd(const void* attn, int64_t ld_attn, const void* out_bias, const void* packed_out_weights,
                          const void* residual, int64_t ldr, const void* norm_weight, float eps, const void* b_up,
                          const void* b_down, const void* packed_ffn_weights, void* out, int64_t ldo, int64_t M,
                          int32_t D, int32_t F, const int32_t* rows, const int32_t* n_rows, const int32_t* attn_rows,
                          int norm_folded, void* stream);

/*
 * The packed q | k | v projection and the block's second half on PER-HEAD PLANES: between the projection, the attention
 * kernel and the out projection a tensor [M, N] may be kept as a stack of N / head_dim planes [M, head_dim] - element
 * (row, col) at ((col / head_dim) * M + row) * head_dim + col % head_dim - so that the rows of one head are contiguous
 * (64 or 128 bytes apart instead of pieces of a 3 * D row): the attention kernel, which takes any strides, then runs 8 %
 * faster at the headline shape, and the dense kernels address the planes at no cost. head_dim = 32 or 64.
 *   taac_norm_linear_heads_fwd: taac_norm_linear_fwd for packed weights without residual whose output is such a stack
 *     (N / head_dim planes; q = planes 0 .. H-1, k = H .. 2H-1, v = 2H .. 3H-1 of a packed projection: pass them to
 *     taac_flash_attn_fwd as base pointers H * M * head_dim elements apart with strides {T * head_dim, M * head_dim,
 *     head_dim, 1}, and let it write its output with the same strides).
 *   taac_attn_out_ffn_heads_fwd: taac_attn_out_ffn_fwd whose attention output `attn` is such a stack of D / head_dim
 *     planes (rows indexed like residual / out: no attn_rows).
 * Results are bit-identical to the row-major entry points. taac_backbone_fwd keeps its q | k | v and attention-output
 * workspace this way for plain attention layers. Replaces: as taac_norm_linear_fwd / taac_attn_out_ffn_fwd; the layout
 * takes the place of the reference's q / k / v transposes to (B, H, T, d) (modeling/sequence.py:100-116).
 */
int taac_norm_linear_heads_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* bias,
                               const void* packed_weights, void* out, int32_t head_dim, int64_t M, int32_t N, int32_t K,
                               const int32_t* rows, const int32_t* n_rows, int norm_folded, void* stream);
int taac_attn_out_ffn_heads_fwd(const void* attn, int32_t head_dim, const void* out_bias, const void* packed_out_weights,
                                const void* residual, int64_t ldr, const void* norm_weight, float eps, const void* b_up,
                                const void* b_down, const void* packed_ffn_weights, void* out, int64_t ldo, int64_t M,
                                int32_t D, int32_t F, const int32_t* rows, const int32_t* n_rows, int norm_folded,
                                void* stream);

/*
 * taac_attn_out_ffn_fwd with a sigmoid gate on the projected update (TokenFormer's NLIR gate):
 *   x1  = residual + sigmoid(update_gate) * (attn @ w_out^T + out_bias)
 *   out = x1 + down( silu(g) * u ) + b_down,   g, u = chunk2( up( norm_weight ? rmsnorm(x1, norm_weight, eps) : x1 ) )
 * update_gate: [M, D] bf16 (row stride ld_gate, rows laid out like residual / out), the gate layer's output BEFORE the
 * sigmoid: nlir_gate(attn_norm(tokens)), e.g. from taac_norm_linear_fwd on the block input. Roundings follow the
 * reference's 16-bit evaluation: the projection, the sigmoid, their product and the sum with the residual are each
 * rounded to bf16. Everything else as in taac_attn_out_ffn_fwd.
 * Replaces: nlir_gate's sigmoid, the gated residual update and ffn_norm + SwiGLUFeedForward.forward + residual add of
 * TokenFormerBlock.forward (experiments/tokenformer/model.py:209-214); the `* valid` factors of that forward are the
 * row index (padded rows are never touched).
 */
int taac_attn_out_gate_ffn_fwd(const void* attn, int64_t ld_attn, const void* out_bias, const void* packed_out_weights,
                               const void* update_gate, int64_t ld_gate, const void* residual, int64_t ldr,
                               const void* norm_weight, float eps, const void* b_up, const void* b_down,
                               const void* packed_ffn_weights, void* out, int64_t ldo, int64_t M, int32_t D, int32_t F,
                               const int32_t* rows, const int32_t* n_rows, const int32_t* attn_rows,
                               int norm_folded, void* stream);

/*
 * Fused [RMSNorm ->] dense layer [-> + residual] with the token rows held in registers:
 *   out = (residual ? residual : 0) + (norm_weight ? rmsnorm(x, norm_weight, eps) : x) @ w^T + bias
 * x: [M, K] bf16; w: [N, K]; bias: [N] or NULL; residual / out: [M, N]; packed_weights: NULL or the blob written by
 * taac_linear_pack_weights for w. K must be 128 or 256, N a multiple of 64. out may alias residual, not x.
 * rows / n_rows: as in taac_swiglu_ffn_fwd (rows of residual and out). x_rows: NULL, or (with rows) the row of x that
 * holds token i when x is laid out differently from residual / out (taac_front_rows).
 * norm_folded != 0 (needs norm_weight and packed_weights): packed_weights is the blob of taac_linear_pack_weights_norm
 * for (w, norm_weight), i.e. the norm's weight is already part of the layer. The kernel then leaves the rows as they
 * are and multiplies its fp32 accumulators by the token's rsqrt(mean(x^2) + eps) before bias and rounding
 * (linear(x * r * g) = r * linear_g(x)): the normalised rows are never formed, which saves about five vector
 * instructions per input element; the result differs from the unfolded form by roundings only (g is rounded into the
 * weights instead of into the rows; exactly equal for g = 1).
 * Replaces: attn_norm + the qkv projection, and the out projection + residual add, of UnifiedInteractionBlock /
 * UnifiedSelfAttention (experiments/symbiosis/backbone.py:34-35, 47, 64-65).
 */
int taac_norm_linear_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w,
                         const void* bias, const void* packed_weights, const void* residual, int64_t ldr, void* out,
                         int64_t ldo, int64_t M, int32_t N, int32_t K, const int32_t* rows, const int32_t* n_rows,
                         const int32_t* x_rows, int norm_folded, void* stream);

/*
 * Query / key preparation of the attention layers, one pass over q and k (each read once, written once; in place when
 * q_out == q and k_out == k):
 *   x_hat = x * rsqrt(mean(x^2 over all d_model features) + eps) * weight      (when q_weight / k_weight are given)
 *   per head, feature pair (2i, 2i+1) at sequence position t:                    (when cos_sin is given)
 *     out[2i]   = x_hat[2i] * cos(t, i) - x_hat[2i+1] * sin(t, i)
 *     out[2i+1] = x_hat[2i] * sin(t, i) + x_hat[2i+1] * cos(t, i)
 * fp32 arithmetic, one rounding to the storage dtype. q, k: [rows, d_model] with row stride ld_in (elements), row r is
 * the token at position r % tokens_per_sample of sample r / tokens_per_sample; q_out, k_out likewise with ld_out.
 * q_weight, k_weight: [d_model] in the storage dtype, both or neither. cos_sin: [tokens_per_sample, head_dim / 2, 2] =
 * (cos, sin) of position * rope_base^(-2i / head_dim), in the storage dtype, or null. row_index / n_rows: optional
 * device-side list of the rows to process (taac_valid_rows), both or neither; other rows are left untouched.
 * d_model, the strides and (with a table) head_dim must be multiples of the 16-byte vector (8 elements, 4 for fp32).
 * Replaces: query_norm / key_norm (RMSNorm(d_model)) of UnifiedSelfAttention.forward
 * (experiments/symbiosis/backbone.py:33-36) and BFTSAttention.forward + _apply_rope + _rotate_half_pairs
 * (experiments/tokenformer/model.py:131-136, 149-154, 165-192), i.e. two norm passes and the elementwise rotary passes.
 */
int taac_qk_norm_rope_fwd(const void* q, const void* k, int64_t ld_in, void* q_out, void* k_out, int64_t ld_out,
                          int64_t rows, int32_t tokens_per_sample, int32_t d_model, int32_t num_heads,
                          const void* q_weight, const void* k_weight, float eps, const void* cos_sin,
                          const int32_t* row_index, const int32_t* n_rows, int dtype, void* stream);

/*
 * taac_norm_linear_fwd for the packed [q | k | v] projection of an attention layer (N = 3 * d_model, K = d_model, no
 * residual) with the query / key preparation folded into the epilogue. For the 2 * d_model query and key features:
 *   qk_sumsq[c, r] = sum of squares of the 64 rounded projection values of chunk c (features 64c .. 64c+63) of row r
 *                    (fp32 [2 * d_model / 64, M]; the statistic of RMSNorm(d_model) is the sum over a projection's
 *                    chunks, see taac_row_rstd), when qk_sumsq is given;
 *   out = rotate(projection * qk_weight) with qk_weight [2 * d_model] = query | key norm weights (NULL: ones) and the
 *         rotation of taac_qk_norm_rope_fwd over cos_sin [tokens_per_sample, head_dim / 2, 2] (NULL: none); row r is
 *         the token at position r % tokens_per_sample.
 * The value features are stored unchanged. The per-token factor rsqrt(mean + eps) of the norm commutes with the weight
 * and the rotation and is left to the attention kernel (taac_flash_attn_scaled_fwd). d_model: 128 or 256; head_dim a
 * multiple of 8 with a table. Other arguments (norm_folded included) as taac_norm_linear_fwd; with x_rows the statistic is indexed by the row
 * of out and the position is that of the row of x.
 * Replaces: qkv + query_norm + key_norm of UnifiedSelfAttention.forward (experiments/symbiosis/backbone.py:33-36)
 * and BFTSAttention._apply_rope (experiments/tokenformer/model.py:165-192) without a pass of their own over q and k.
 */
int taac_norm_linear_qk_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w,
                            const void* bias, const void* packed_weights, void* out, int64_t ldo, int64_t M,
                            int32_t d_model, int32_t num_heads, int32_t tokens_per_sample, const void* qk_weight,
                            const void* cos_sin, float* qk_sumsq, const int32_t* rows, const int32_t* n_rows,
                            const int32_t* x_rows, int norm_folded, void* stream);

/*
 * rstd[0, r] = rsqrt(sum_c qk_sumsq[c, r] / d_model + eps) over the d_model / 64 chunks of the query projection,
 * rstd[1, r] likewise over the key projection's chunks: fp32 [2, M], the q_row_scale / k_row_scale of
 * taac_flash_attn_scaled_fwd. With rows / n_rows only the listed rows are written.
 */
int taac_row_rstd(const float* qk_sumsq, int64_t M, int32_t d_model, float eps, float* rstd, const int32_t* rows,
                  const int32_t* n_rows, void* stream);

/*
 * Readout of the token backbone, one kernel:
 *   n(t)  = token_norm_weight ? rmsnorm(tokens[b, t], token_norm_weight, eps) : tokens[b, t]
 *   e[b]  = concat( n(cls_index), candidate_index >= 0 ? n(candidate_index) : 0, mean over the valid t of n(t) )
 *   e[b]  = pool_norm_weight ? rmsnorm(e[b], pool_norm_weight, eps) : e[b]                       [3D]
 *   z[b]  = fc2( silu( fc1(e[b]) ) ),  optionally sigmoid(z[b])                                  [actions]
 * tokens: [B, T, D] bf16 contiguous. Valid tokens: t < key_lengths[b] (clamped to [0, T]) when key_lengths is given,
 * bit t of valid_bits[b] (rows of ceil(T / 32) 32-bit words, as written by taac_mask_pack_bits from a [B, T] bool
 * matrix, True = valid) when valid_bits is given, every token when both are NULL; the mean's divisor is clamped to
 * >= 1 (modeling/sequence.py:54-60). The cls and candidate tokens are taken whether valid or not, as the reference
 * does. fc1_weight: [hidden, 3D], fc2_weight: [actions, hidden] (torch nn.Linear layout), biases may be NULL;
 * fc1_weight NULL skips the classifier. embedding_out: [B, 3D] bf16 or NULL; logits_out: [B, actions] fp32 (required
 * with a classifier). D a multiple of 8, D and hidden at most 1024. Evaluated in fp32 from the stored operands.
 * Replaces: final_norm + CandidateClsPooler.forward + classifier of PCVRSymbiosis (experiments/symbiosis/model.py:
 * 215-222, 291, 309, 316-317; experiments/symbiosis/pooling.py:16-32).
 */
int taac_candidate_readout_fwd(const void* tokens, const int32_t* key_lengths, const uint32_t* valid_bits, int32_t B,
                               int32_t T, int32_t D, int32_t cls_index, int32_t candidate_index,
                               const void* token_norm_weight, const void* pool_norm_weight, float eps,
                               const void* fc1_weight, const void* fc1_bias, int32_t hidden, const void* fc2_weight,
                               const void* fc2_bias, int32_t actions, void* embedding_out, float* logits_out,
                               int apply_sigmoid, void* stream);

/*
 * Row index of the valid tokens of a padded batch: token t of sample b is valid iff t < key_lengths[b] (clamped to
 * [0, T]). Writes rows[i] = b * T + t for the valid tokens in increasing order, *n_rows = their number, and the
 * per-sample offsets (exclusive prefix sums of the lengths, B + 1 values, the last one equal to *n_rows) to
 * rows[B * T .. B * T + B]. rows must hold B * T + B + 1 values. Everything stays on the device.
 * No counterpart in the reference, which runs its dense layers over the padded positions as well
 * (experiments/symbiosis/backbone.py:58-68 masks their updates afterwards).
 */
int taac_valid_rows(const int32_t* key_lengths, int32_t B, int32_t T, int32_t* rows, int32_t* n_rows, void* stream);

/*
 * dst[i, 0..W) = src[rows[i], 0..W) for i < n: rows of 16-bit elements (W a multiple of 8; src row stride ld_src elements,
 * dst contiguous). With the index of taac_valid_rows and n = the number of valid rows it compacts the valid tokens of a
 * padded [B * T, W] tensor. No counterpart in the reference (torch.index_select in its place).
 */
int taac_rows_gather(const void* src, int64_t ld_src, const int32_t* rows, int64_t n, void* dst, int32_t W, void* stream);

/*
 * Merge of a padded and a compact layout (bf16 rows of W elements, W a multiple of 8): row (b, t) of out [B * T, W] is
 * compact_a[offsets[b] + t] (+ compact_b of the same row when compact_b is not NULL; fp32 add, one rounding) for
 * t < key_lengths[b], and the row of `padded` otherwise. offsets: the per-sample offsets taac_valid_rows writes behind
 * its row index (rows + B * T). out may be `padded`.
 * Replaces: the scatter of a valid-row gradient (or output) into the padded token stream that
 * `update * ~padding_mask` + residual adds amount to in UnifiedInteractionBlock (experiments/symbiosis/backbone.py:58-68).
 */
int taac_rows_merge(const void* padded, const void* compact_a, const void* compact_b, const int32_t* key_lengths,
                    const int32_t* offsets, void* out, int32_t B, int32_t T, int32_t W, void* stream);

/*
 * taac_flash_attn_mask_bwd with the mask in the bit form of taac_flash_attn_masked_train_fwd: struct_bits rows of
 * ceil(Tk / 32) words per query (struct_sample_stride words between the matrices of consecutive samples, 0 = one matrix
 * for the batch), valid_bits [B, ceil(Tk / 32)] or NULL; pair (i, j) of sample b is visible iff both bits are set (and
 * j < key_lengths[b] when key_lengths is given). One word per 32-key tile where the byte form reads 32 bytes. With the
 * samples' valid tokens at the front of their rows (taac_front_rows, taac_mask_front_bits) and key_lengths = their
 * numbers, the cost follows the valid tokens as in taac_flash_attn_bwd. dropout_mask (NULL: none): the keep mask and
 * scale of the forward, as in taac_flash_attn_dropout_bwd.
 * Replaces: as taac_flash_attn_mask_bwd; with dropout, what the reference's models train with by default
 * (experiments/symbiosis/__init__.py:87).
 */
int taac_flash_attn_bits_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout, const float* lse,
                             const int32_t* key_lengths, const uint32_t* struct_bits, int64_t struct_sample_stride,
                             const uint32_t* valid_bits, const uint8_t* dropout_mask, float dropout_scale, void* dq,
                             void* dk, void* dv, float* delta, int32_t B, int32_t H,
                             int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4], const int64_t k_strides[4],
                             const int64_t v_strides[4], const int64_t o_strides[4], const int64_t do_strides[4],
                             const int64_t dq_strides[4], const int64_t dk_strides[4], const int64_t dv_strides[4],
                             int zero_padded_queries, int dtype, void* stream);

/*
 * taac_rows_merge for padding that is not a prefix: token t of sample b is valid iff bit t of valid_bits[b] is set (rows
 * of ceil(T / 32) words, as for taac_valid_rows_from_bits, whose per-sample offsets are `offsets`); its compact row is
 * offsets[b] + the number of valid tokens of the sample in front of it. word_prefix (NULL: the kernel counts): int32
 * [B, ceil(T / 32)], the number of valid tokens of the sample in the words before each word.
 * Replaces: the same `update * ~padding_mask` + residual arithmetic under the scattered padding of the reference's
 * token layout (experiments/symbiosis/backbone.py:58-68, experiments/symbiosis/attention.py:21-60).
 */
int taac_rows_merge_bits(const void* padded, const void* compact_a, const void* compact_b, const uint32_t* valid_bits,
                         const int32_t* word_prefix, const int32_t* offsets, void* out, int32_t B, int32_t T, int32_t W,
                         void* stream);

/*
 * The same row index for padding that is not a prefix: token t of sample b is valid iff bit t of valid_bits[b] is set
 * (rows of ceil(T / 32) 32-bit words, as written by taac_mask_pack_bits from a [B, T] bool matrix, True = valid).
 * Output layout and sizes as in taac_valid_rows. This is what lets the dense layers honour the reference blocks'
 * `update * ~padding_mask` (experiments/symbiosis/backbone.py:65, 67) by not touching the padded rows at all.
 */
int taac_valid_rows_from_bits(const uint32_t* valid_bits, int32_t B, int32_t T, int32_t* rows, int32_t* n_rows,
                              void* stream);

/*
 * Second row index for a layout in which every sample's valid tokens sit at the front of its T rows, in their
 * original order: front_rows[i] = b * T + (rank of token i among the valid tokens of its sample b), for the tokens of
 * a row index written by taac_valid_rows / taac_valid_rows_from_bits (rows, with its offsets in rows[B * T ..]), and
 * lengths[b] = number of valid tokens of sample b. A projection that reads x through rows and writes through
 * front_rows (taac_norm_linear_fwd / taac_norm_linear_qk_fwd with rows = front_rows, x_rows = rows) turns scattered
 * padding into prefix padding for the attention call (key_lengths = lengths, zero_padded_queries = 2), whose cost then
 * follows the valid tokens instead of T; the out projection reads it back through attn_rows / x_rows = front_rows.
 * front_rows holds B * T values, lengths B. No counterpart in the reference, whose attention visits every position.
 */
int taac_front_rows(const int32_t* rows, const int32_t* n_rows, int32_t B, int32_t T, int32_t* front_rows,
                    int32_t* lengths, void* stream);

/*
 * A structural mask in that front layout: out_bits[b, r, :] (rows of ceil(T / 32) words, T rows per sample) holds, for
 * the r-th valid token of sample b, bit j = struct_bits[position(b, r), position(b, j)] for j below the sample's
 * number of valid tokens n_b and zeros up to the end of the 64-key group of key n_b - 1. Nothing else is written (rows
 * at or beyond n_b, words beyond that group): the attention call below does not read it. struct_bits:
 * [T, ceil(T / 32)] (taac_mask_pack_bits), rows: the index of taac_valid_rows_from_bits. Use with key_lengths =
 * the lengths of taac_front_rows, zero_padded_queries = 1 or 2, struct_sample_stride = T * ceil(T / 32) and
 * valid_bits = block_any = NULL in taac_flash_attn_masked_fwd. T <= 4096.
 */
int taac_mask_front_bits(const uint32_t* struct_bits, int32_t T, const int32_t* rows, int32_t B, uint32_t* out_bits,
                         void* stream);

/*
 * Weight packing for the two fused kernels above: copies the weights into MFMA-fragment order (the order in which
 * the kernels stage them into LDS). Pack once per weight set; the blob has the size of the weights themselves.
 * The FFN blob depends on gate_first (which half of w_up is gated): taac_swiglu_ffn_fwd must be given the same value.
 * taac_*_packed_bytes return the blob size, or -1 for shapes the fused kernels do not take.
 * No counterpart in the reference (its dense layers are library GEMMs on nn.Linear weights).
 */
int64_t taac_ffn_packed_bytes(int32_t D, int32_t F);
int taac_ffn_pack_weights(const void* w_up, const void* w_down, void* packed, int32_t D, int32_t F, int gate_first,
                          void* stream);
/* The same blob with the weight of the RMSNorm in front of the up projection folded into its fragments
 * (w_up[n, k] * norm_weight[k], rounded once), for the feed-forward entry points with norm_folded = 1. */
int taac_ffn_pack_weights_norm(const void* w_up, const void* w_down, const void* norm_weight, void* packed, int32_t D,
                               int32_t F, int gate_first, void* stream);
/* The same blob (norm_weight: NULL, or folded as above) which, with fold_activation != 0, also carries the constants of
 * the gate's activation: the gated half of the up projection is multiplied by -log2(e) and the other half by -ln(2)
 * inside the same single rounding of each weight, so that silu(g) * u = g' * u' / (1 + 2^g') with g', u' as the matrix
 * unit delivers them - one multiplication less per hidden unit and token in the kernels, which are then called with
 * TAAC_FOLDED_ACTIVATION in norm_folded (they scale b_up the same way when they stage it).
 * taac_ffn_activation_fold_supported: 1 where the kernels take such a blob (D 128 / 256, F a multiple of 32 that leaves
 * room for three weight buffers), else 0. No counterpart in the reference. */
#define TAAC_FOLDED_NORM 1
#define TAAC_FOLDED_ACTIVATION 2
int taac_ffn_activation_fold_supported(int32_t D, int32_t F);
int taac_ffn_pack_weights_folded(const void* w_up, const void* w_down, const void* norm_weight, void* packed, int32_t D,
                                 int32_t F, int gate_first, int fold_activation, void* stream);
int64_t taac_linear_packed_bytes(int32_t N, int32_t K);
int taac_linear_pack_weights(const void* w, void* packed, int32_t N, int32_t K, void* stream);
/* The same blob with the weight of an RMSNorm in front of the layer folded in (packed[n, k] = bf16(w[n, k] *
 * norm_weight[k])), for taac_norm_linear_fwd / taac_norm_linear_qk_fwd with norm_folded = 1. */
int taac_linear_pack_weights_norm(const void* w, const void* norm_weight, void* packed, int32_t N, int32_t K, void* stream);

/*
 * Per-tensor absolute maximum, for the FP8 scale (scale = amax / 448). Writes max(|x|) over n elements to
 * *amax_out (device float). The kernel clears *amax_out itself before reducing.
 * No counterpart in the reference (it has no FP8 code); defined by the FP8 configuration of this path.
 */
int taac_amax(const void* x, int64_t n, int dtype, float* amax_out, void* stream);

/*
 * Quantise to OCP e4m3fn with a per-tensor scale: q = sat(x / scale) where scale = max(*amax, tiny) / 448.
 * x: n elements of `dtype`; q: n bytes; amax: device float. Round-to-nearest-even, saturating at +-448.
 */
int taac_quantize_fp8(const void* x, int64_t n, int dtype, const float* amax, void* q, void* stream);

/*
 * Dense layer with FP8 (e4m3fn) MFMA operands and per-tensor scales:
 *   out = epilogue( (qa @ qw^T) * (amax_a / 448) * (amax_w / 448) + bias )
 * a: [M, K] bf16 activations, quantised on load with scale amax_a / 448 (a_is_fp8 == 0), or already e4m3
 * bytes (a_is_fp8 != 0). w: [N, K] e4m3 bytes. amax_a / amax_w: device floats. bias / residual / out are bf16
 * with the same meaning as in taac_linear_bf16. K must be a multiple of 16.
 * No counterpart in the reference; semantics follow the quantize -> matmul -> dequantize emulation
 * q = (t / s).to(float8_e4m3fn), y = (qa.float() @ qw.float().T) * s_a * s_w.
 */
int taac_linear_fp8(const void* a, int a_is_fp8, int64_t lda, const void* w, const float* amax_a, const float* amax_w,
                    const void* bias, const void* residual, void* out, int64_t ldo, int64_t M, int32_t N, int32_t K,
                    int epilogue, int gate_first, void* stream);

/*
 * Fused [RMSNorm ->] FP8 dense layer [-> + residual], the FP8 counterpart of
 * taac_norm_linear_fwd (K = 256, N a multiple of 64):
 *   h   = norm_weight ? bf16(rmsnorm(x, norm_weight, eps)) : x                    quantised with scale amax_x / 448
 *   out = bf16( (q(h) q(w)^T) (amax_x / 448)(amax_w / 448) + bias [+ residual] )  one rounding
 * x: [M, K] bf16 (row stride ldx); w_fp8: [N, K] e4m3 bytes (taac_quantize_fp8 with amax_w); amax_x: max |h| over the
 * tokens (device float; of the normalised rows when norm_weight is given). rows / n_rows: as in taac_swiglu_ffn_fwd
 * (token i lives in row rows[i] of x / residual / out; other rows are neither read nor written).
 * amax_out (or NULL): receives the per-tensor scale of the layer that consumes out, reduced in the epilogue (no pass of
 * its own): max over the tokens of | bf16( rstd * max_f |out_f * out_norm_weight_f| ) | with rstd the RMSNorm statistic
 * of the rounded output row (eps out_eps), or max |out| when out_norm_weight is NULL. The first form equals
 * max | bf16(rmsnorm(out, out_norm_weight)) | up to the order of two fp32 multiplications.
 * No counterpart in the reference (it has no FP8 code).
 */
int taac_norm_linear_fp8_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w_fp8,
                             const void* bias, const float* amax_x, const float* amax_w, const void* residual, int64_t ldr,
                             void* out, int64_t ldo, int64_t M, int32_t N, int32_t K, const int32_t* rows,
                             const int32_t* n_rows, const void* out_norm_weight, float out_eps, float* amax_out,
                             void* stream);

/*
 * Fused feed-forward half with FP8 (e4m3fn) MFMA operands and per-tensor scales, the FP8 counterpart of
 * taac_swiglu_ffn_fwd: the chain of two taac_linear_fp8 layers
 *   h   = norm_weight ? bf16(rmsnorm(x, norm_weight, eps)) : x
 *   hid = silu(g) * u,  g, u = chunk2( (q(h) q(w_up)^T) (amax_x / 448)(amax_up / 448) + b_up )      (kept in fp32)
 *   out = bf16( (q(hid) q(w_down)^T) (amax_hidden / 448)(amax_down / 448) + b_down + residual )
 * with q(t) = sat(t / (amax_t / 448)) in e4m3 and amax_hidden = max |hid| over all tokens, which the call computes
 * itself: a first launch evaluates the up projection and the gate only to reduce max |hid| into *amax_hidden, a second
 * launch evaluates the whole layer with that scale. The [M, F] hidden state is never written to memory, so it is
 * quantised from fp32 (the chain of two separate layers rounds it to bf16 in between: a difference of at most one bf16
 * step before a quantisation to three mantissa bits).
 * packed_weights: blob of taac_ffn_fp8_pack_weights (both weights quantised with their amax and laid out in fragment
 * order; 3 * D * F + 64 * D bytes, taac_ffn_fp8_packed_bytes). amax_x: device float, max |h| over the tokens (of the normalised
 * input when norm_weight is given: taac_amax of it, or the amax_next / amax_out of the producing call). amax_up /
 * amax_down: the amax the weights were packed with. amax_hidden: device float, written. x, residual, out, rows / n_rows,
 * gate_first: as in taac_swiglu_ffn_fwd (out may alias residual and x). D: 128 or 256, F a multiple of 64.
 * amax_next (or NULL): receives max | bf16(rmsnorm(out, next_norm_weight, next_eps)) | over the tokens (max |out| when
 * next_norm_weight is NULL): the amax_x of the layer that consumes out, so that no pass of its own is needed for it.
 * No counterpart in the reference (it has no FP8 code); semantics follow the quantize -> matmul -> dequantize emulation.
 */
int64_t taac_ffn_fp8_packed_bytes(int32_t D, int32_t F);
int taac_ffn_fp8_pack_weights(const void* w_up, const void* w_down, const float* amax_up, const float* amax_down,
                              void* packed, int32_t D, int32_t F, int gate_first, void* stream);
int taac_swiglu_ffn_fp8_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* packed_weights,
                            const void* b_up, const void* b_down, const float* amax_x, const float* amax_up,
                            const float* amax_down, float* amax_hidden, const void* residual, int64_t ldr, void* out,
                            int64_t ldo, int64_t M, int32_t D, int32_t F, int gate_first, const int32_t* rows,
                            const int32_t* n_rows, const void* next_norm_weight, float next_eps, float* amax_next,
                            void* stream);

/*
 * Readout of the backbone: p[b] = sigmoid( masked_mean(x[b, :L_b, :]) . w_head + b_head ), with
 * L_b = clamp(lengths[b], 0, T) and the mean's divisor clamped to >= 1.
 * x: [B, T, D] bf16 contiguous; lengths: int32 [B]; w_head: [D] bf16; b_head: [1] bf16 or NULL; p: float [B].
 * Replaces: masked_mean (infrastructure/modeling/sequence.py:54-60) followed by Linear(D, 1) and sigmoid.
 */
int taac_masked_mean_head(const void* x, const int32_t* lengths, const void* w_head, const void* b_head, float* p,
                          int32_t B, int32_t T, int32_t D, void* stream);

/*
 * Multi-hot embedding lookup with mean pooling: out[b, :] = mean of weight[id, :] over the ids of bag b that are not the
 * padding id 0; a bag without any such id gives zeros. fp32 accumulation, one rounding to the table's dtype.
 * weight: [num_embeddings, emb_dim] contiguous; values: [bags, bag_size] int32 (index_is_int64 == 0) or int64,
 * contiguous; out: [bags, emb_dim] in weight's dtype. Ids outside [0, num_embeddings) are skipped like padding and, when
 * invalid_count (one int32 on the device, zeroed by the caller) is given, counted there: the reference's torch backend
 * raises an index error for them, a caller that wants that behaviour reads the counter.
 * Replaces: embedding_bag_mean / _torch_embedding_bag_mean = F.embedding_bag(values, weight, mode="mean",
 * padding_idx=0) (src/taac2026/infrastructure/accelerators/embedding/embedding_bag.py:82-83, 439-467), the step that
 * feeds the token backbone (infrastructure/modeling/embeddings.py:65-71); same signature as a kernel registered
 * through register_embedding_bag_mean_kernel (embedding_bag.py:39,77-79).
 */
int taac_embedding_bag_mean_fwd(const void* weight, int64_t num_embeddings, int32_t emb_dim, const void* values,
                                int index_is_int64, int64_t bags, int32_t bag_size, void* out, int32_t* invalid_count,
                                int dtype, void* stream);

/*
 * Gradient of the table under taac_embedding_bag_mean_fwd: grad_weight[id, :] = sum over the bags b and their slots j
 * with values[b, j] == id of grad_out[b, :] / max(count_b, 1), count_b = the number of ids of bag b that are neither the
 * padding id 0 nor outside [0, num_embeddings); rows no bag names are zero. The whole [num_embeddings, emb_dim] gradient
 * is written (it is cleared here, not by the caller). Sums are formed in fp32 by float add-to-memory, so a row named
 * by several bags adds in an order that may differ from launch to launch (last-bit differences, as with the
 * reference's atomic adds); a 16-bit table needs workspace = num_embeddings * emb_dim floats (16-byte aligned) for
 * those sums and is rounded once at the end, an fp32 table is accumulated in place (workspace may be NULL).
 * values: [bags, bag_size] int32 / int64 contiguous; grad_out: [bags, emb_dim] contiguous in the table's dtype;
 * grad_weight: [num_embeddings, emb_dim] in the table's dtype.
 * Replaces: the embedding-bag mean backward kernels (src/taac2026/infrastructure/accelerators/embedding/kernels/
 * triton.py:91-150, tilelang.py:95-140) called from the autograd functions' backward (embedding_bag.py:345-353).
 */
int taac_embedding_bag_mean_bwd(const void* values, int index_is_int64, int64_t bags, int32_t bag_size,
                                const void* grad_out, void* grad_weight, int64_t num_embeddings, int32_t emb_dim,
                                void* workspace, int dtype, void* stream);

/*
 * Weights of one backbone block; every pointer is a device pointer to bf16 data in torch nn.Linear layout.
 * Field names follow the reference's parameter names (experiments/symbiosis/backbone.py:24-56).
 * Biases may be NULL (treated as zero). query_norm_weight / key_norm_weight are the attention layer's
 * RMSNorm(d_model) of its query and key (backbone.py:30-36); NULL gives the plain layer of the benchmark recipe.
 */
typedef struct taac_block_weights {
  const void* attn_norm_weight; /* [D]                                   */
  const void* qkv_weight;       /* [3D, D], rows ordered q, k, v         */
  const void* qkv_bias;         /* [3D]                                  */
  const void* out_weight;       /* [D, D]                                */
  const void* out_bias;         /* [D]                                   */
  const void* ffn_norm_weight;  /* [D]                                   */
  const void* up_weight;        /* [2F, D], rows ordered gate, value     */
  const void* up_bias;          /* [2F]                                  */
  const void* down_weight;      /* [D, F]                                */
  const void* down_bias;        /* [D]                                   */
  const void* query_norm_weight; /* [D] RMSNorm(d_model) of the query projection, or NULL: no query / key norm */
  const void* key_norm_weight;   /* [D] likewise for the key projection (both or neither)                       */
} taac_block_weights;

/* Bytes of workspace taac_backbone_fwd needs for the given shape (device memory, 256-byte aligned): activations
 * plus, for the fused path, one fragment-ordered copy of every block's weights (repacked on each call). */
int64_t taac_backbone_workspace_bytes(int32_t B, int32_t T, int32_t D, int32_t F, int32_t n_blocks);

/* Byte offset, inside the workspace of taac_backbone_fwd, of the per-tensor maxima a TAAC_BACKBONE_FP8 call leaves
 * behind: float [n_blocks + 1][8] = per block {|w_qkv|, |w_out|, |w_up|, |w_down|, |rmsnorm(x)|, |attention|,
 * |rmsnorm(x1)|, |silu(gate) * value|} (scale = maximum / 448); the last row holds nothing. -1 when the shape has no
 * FP8 mode. No counterpart in the reference (its FP8 layers keep the scales inside the layer); for calibration and
 * tests. */
int64_t taac_backbone_fp8_scales_offset(int32_t B, int32_t T, int32_t D, int32_t F, int32_t n_blocks);

/*
 * Forward of n_blocks pre-norm blocks plus the pCVR readout:
 *   for each block: h = rmsnorm(x); q,k,v = chunk3(h Wqkv^T + b);
 *                   [q = rmsnorm(q, query_norm_weight); k = rmsnorm(k, key_norm_weight) over all D features]
 *                   [q, k = rotary embedding over the token positions, table rope_cos_sin]
 *                   a = attention(q,k,v, key_lengths)
 *                   (padded query rows -> 0); x = x + a Wo^T + b; h2 = rmsnorm(x);
 *                   g,u = chunk2(h2 Wup^T + b); x = x + (silu(g) * u) Wdown^T + b
 *   p = sigmoid(masked_mean(x, lengths) . w_head + b_head)
 * emb: [B, T, D] bf16 (not modified); key_lengths: int32 [B] valid-prefix lengths; hidden_out: [B, T, D] bf16
 * final hidden state or NULL; p: float [B]. heads divides D and D / heads is a multiple of 8.
 * rope_cos_sin: [T, D / heads / 2, 2] bf16 table of (cos, sin) as in taac_qk_norm_rope_fwd, or NULL (no rotation);
 * the same eps serves every norm. flags: TAAC_BACKBONE_* bits, 0 for the default route (the dense layers skip the
 * padded positions; rows at or beyond key_lengths[b] of hidden_out are then zeros, with TAAC_BACKBONE_DENSE_TOKENS they
 * hold the values the dense formulation computes there; the readout never reads them). With TAAC_BACKBONE_FP8 every
 * dense layer is the quantize -> matmul -> dequantize layer of taac_linear_fp8 (weights quantised per call; every
 * activation scale is the exact per-tensor maximum, reduced in the epilogue of the kernel that produces the tensor:
 * taac_norm_linear_fp8_fwd, taac_flash_attn_amax_fwd, taac_swiglu_ffn_fp8_fwd).
 * Replaces: the block loop _run_backbone (experiments/symbiosis/model.py:283-292) over UnifiedInteractionBlock
 * (experiments/symbiosis/backbone.py:50-68) in its canonical pre-norm form, plus masked_mean + Linear + sigmoid; with
 * the query / key norm weights UnifiedSelfAttention as the reference runs it (backbone.py:24-48), with the table
 * TokenFormer's BFTSAttention (experiments/tokenformer/model.py:139-192).
 */
int taac_backbone_fwd(const void* emb, const int32_t* key_lengths, const taac_block_weights* blocks, int32_t n_blocks,
                      const void* w_head, const void* b_head, int32_t B, int32_t T, int32_t D, int32_t heads, int32_t F,
                      float eps, const void* rope_cos_sin, int flags, void* workspace, int64_t workspace_bytes,
                      void* hidden_out, float* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TAAC_HIP_H */

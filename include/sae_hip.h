/*
 * sae_hip.h -- C ABI of libsae_hip.so: the sparse-autoencoder train step on MI355X (gfx950).
 *
 * Conventions (all entry points):
 *   - plain device pointers, 64-bit sizes, a dtype enum and a hipStream_t passed as void*;
 *   - return 0 on success, a negative SAE_ERR_* code otherwise; sae_last_error() then
 *     returns a thread-local, human-readable message;
 *   - nothing here allocates or frees device memory, and nothing synchronises the stream:
 *     outputs and workspaces are caller-owned (sizes from the *_workspace_bytes queries);
 *   - inputs are never modified unless the parameter is documented "in/out".
 *
 * Layout vocabulary:
 *   B tokens, d = d_model, F = d_sae, k = top_k.
 *   "feature-major" = [F, d] row-major: one feature's d_model-vector is contiguous.
 *   The decoder W_D [F, d] is feature-major in the reference already
 *   (src/llamascopium/models/sae.py:69).  The encoder is W_E [d, F] in the reference
 *   (models/sae.py:67); this library consumes its transpose W_E^T [F, d] (feature-major),
 *   i.e. the same memory a [d, F] tensor with strides (1, d) views.
 *
 * Sparse code ("feature activations" in sparse form), produced by the select entry points:
 *   idx     int32  flat array of feature indices,
 *   val     fp32   flat array of feature activations (already divided by the decoder-norm
 *                  scale when one was applied),
 *   row_off int64  [B]  first slot of token b in idx/val,
 *   row_nnz int32  [B]  number of valid slots of token b; indices ascend within a token.
 *   For per-token TopK row_off[b] = b*k and unused slots hold idx 0 / val 0.
 *
 * Each declaration cites the reference code it replaces (paths relative to the reference
 * checkout, src/llamascopium/...).
 */
#ifndef SAE_HIP_H
#define SAE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum { SAE_F32 = 0, SAE_BF16 = 1 } sae_dtype;

enum {
  SAE_OK = 0,
  SAE_ERR_INVALID_ARG = -1,   /* null pointer, non-positive size, bad enum            */
  SAE_ERR_UNSUPPORTED = -2,   /* shape outside what the kernels are built for         */
  SAE_ERR_LAUNCH = -3,        /* hipGetLastError() after a launch                     */
  SAE_ERR_WORKSPACE = -4      /* workspace pointer null or too small                  */
};

/* Library identification and error text. */
int sae_abi_version(void);
const char *sae_last_error(void);

/* ---- element-wise helpers --------------------------------------------------------- */

/* dst[i] = bf16(src[i]) (round-to-nearest-even).  What torch.autocast does to the GEMM
 * operands (trainer.py:613). */
int sae_cast_f32_to_bf16(const float *src, void *dst, int64_t n, void *stream);

/* out[f] = ||W[f, :]||_2 for feature-major W [F, d] fp32.
 * Replaces decoder_norm()/encoder_norm() (models/sae.py:136-160). */
int sae_row_norm(const float *w, float *out, int64_t F, int64_t d, void *stream);

/* dst[c, r] = src[r, c] for fp32 src [rows, cols] -> dst [cols, rows].  Used to import
 * a reference-layout W_E [d, F] into feature-major form and back. */
int sae_transpose_f32(const float *src, float *dst, int64_t rows, int64_t cols, void *stream);

/* out[j] (+)= sum_b src[b, j] for src [B, n] fp32.  accumulate != 0 adds to out.
 * workspace: sae_col_sum_workspace_bytes(B, n) bytes.  The summation order is fixed, so the
 * result is reproducible.  Replaces the bias gradients autograd produces (sum over the
 * token dim). */
int64_t sae_col_sum_workspace_bytes(int64_t B, int64_t n);
int sae_col_sum(const float *src, float *out, int64_t B, int64_t n, int accumulate, void *workspace,
                int64_t workspace_bytes, void *stream);

/* sae_col_sum for callers that cannot allocate a workspace (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The partial sums live in a fixed
 * 4 MiB device array inside the library (one copy per GPU, held until the process ends), so the call allocates
 * nothing; n is limited to SAE_COL_SUM_STATIC_MAX_N columns (larger n: SAE_ERR_UNSUPPORTED; use sae_col_sum).
 * Same kernels and order of additions as sae_col_sum: identical bits.  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (different streams) race; calls on one stream are ordered and safe. */
#define SAE_COL_SUM_STATIC_MAX_N 16384
int sae_col_sum_static(const float *src, float *out, int64_t B, int64_t n, int accumulate, void *stream);

/* ---- encoder ---------------------------------------------------------------------- */

/* pre[b, f] = sum_j x[b, j] * w_enc_t[f, j]          (no bias: the select kernels add it)
 * x [B, d] and w_enc_t [F, d] share in_dtype (SAE_BF16: bf16 operands, fp32 accumulate;
 * SAE_F32: fp32 MFMA).  pre [B, F] is written as out_dtype; SAE_BF16 rounds the fp32
 * accumulator to bf16, which is what the autocast matmul returns.
 * Requires d % 64 == 0 (bf16) / d % 32 == 0 (fp32); B and F arbitrary (edge tiles masked).
 * Replaces `x @ self.W_E` (models/sae.py:324). */
int sae_encoder_gemm(const void *x, const void *w_enc_t, void *pre, int64_t B, int64_t d, int64_t F,
                     int in_dtype, int out_dtype, void *stream);

/* Split-K form of sae_encoder_gemm for bf16 operands: slice s of the contraction axis (d / n_splits elements of every
 * row) gives partials[s] (fp32 [n_splits, B, F]); their sum, which the caller forms in slice order, is the product.  For
 * products with few output tiles and a long contraction (weight gradients over the token axis of a small dictionary),
 * which would otherwise occupy a fraction of the chip.  d % (64 n_splits) == 0. */
int sae_encoder_gemm_split_k(const void *x_bf16, const void *w_t_bf16, float *partials, int64_t n_splits, int64_t B, int64_t d,
                             int64_t F, void *stream);

/* The same bf16 product for operands in either layout: out[m, n] = sum_k A[m, k] B[n, k], fp32 accumulation, out [M, N]
 * written as out_dtype.  a_k_major / b_k_major = 0: the operand is stored [rows, K] (a row's K values side by side, as
 * sae_encoder_gemm takes both); 1: it is stored [K, rows] (K-major: the rows' values side by side), read as it lies, with
 * no transposed copy: its matrix-core fragments are read across the K-rows of the LDS tile.  That is the layout the products
 * over the token axis find their operands in, and the dense decode its weight:
 *   dW_E^T = d(pre)^T x and dW_D = acts^T d(recon)   (autograd of `x @ self.W_E` / `feature_acts @ self.W_D`,
 *            models/sae.py:324, 367): A = d(pre) or acts [tokens, F], B = x or d(recon) [tokens, d], both K-major;
 *   feature_acts @ W_D   (models/sae.py:367):          A = feature_acts [tokens, F], B = W_D [F, d] K-major.
 * n_splits > 1 cuts the contraction into that many slices, run as one launch; out is then fp32 [n_splits, M, N] partial
 * results, to be summed by the caller in slice order.  K % (64 n_splits) == 0; a K-major operand needs its row count
 * (M or N) to be a multiple of 8; pointers 16-byte aligned. */
int sae_gemm_bf16(const void *a, int a_k_major, const void *b, int b_k_major, void *out, int out_dtype, int64_t M, int64_t N,
                  int64_t K, int64_t n_splits, void *stream);

/* ---- activation select ------------------------------------------------------------ */

/* Per-token TopK with fused bias and decoder-norm scale.
 *   h0 = pre[b, f] + b_enc[f]            (b_enc may be null = 0)
 *   h1 = h0 * scale[f]                   (scale may be null = 1; it is ||W_D[f]||)
 *   keep the k largest h1 > 0 of each token; ties -> lowest feature index;
 *   val = h1 / scale (= feature_acts), idx ascending within the token.
 * Outputs idx/val [B, k], row_off [B] (= b*k), row_nnz [B] (<= k; fewer when a token has
 * fewer than k positive pre-activations).
 * Replaces the topk closure (models/sparse_dictionary.py:733-759) + utils/math.py:81-171 and
 * the scale/unscale around it (models/sae.py:334-341). */
int sae_select_topk_row(const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                        int64_t B, int64_t F, int k, int32_t *idx, float *val, int64_t *row_off,
                        int32_t *row_nnz, void *stream);

/* Same, with two more knobs.
 *   feat_mask (nullable, fp32 0/1 [F]): the aux-k form, h1 = ((h0 * scale) / scale) * feat_mask * scale,
 *     i.e. `hidden_pre * is_dead * decoder_norm` op for op (models/sparse_dictionary.py:952-972);
 *   cand_cap (0..4096): capacity of the in-LDS candidate list.  A token whose candidates do not
 *     fit takes the general path (radix histograms over the whole row), which returns the
 *     identical result; cand_cap = 0 forces it for every token (testing and tuning). */
int sae_select_topk_row_ex(const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                           const float *feat_mask, int64_t B, int64_t F, int k, int32_t *idx, float *val, int64_t *row_off,
                           int32_t *row_nnz, int cand_cap, void *stream);

/* sae_select_topk_row for a dictionary whose dtype is bfloat16 (config.py:39): pre is bf16, and the sum with the
 * bias, the product with the scale and the final quotient are each rounded to bf16, as the bf16 tensors
 * `x @ W_E + b_E`, `hidden_pre * decoder_norm()` and `feature_acts / decoder_norm()` are (models/sae.py:324-341).
 * b_enc / scale are fp32 copies of the bf16 bias / norms.  Keys then collide often; ties -> lowest feature index.
 * feat_mask (0/1 per feature, or NULL): the aux-k selection of such a dictionary, whose keys are
 * `hidden_pre * is_dead * decoder_norm` with hidden_pre the bf16 quotient `encode` returned, i.e. two more roundings
 * (models/sparse_dictionary.py:958-970). */
int sae_select_topk_row_lowp(const void *pre_bf16, const float *b_enc, const float *scale, const float *feat_mask,
                             int64_t B, int64_t F, int k, int32_t *idx, float *val, int64_t *row_off, int32_t *row_nnz,
                             void *stream);

/* out[b, f] = bf16(float(bf16(sum_j x[b, j] * w_t[f, j])) + col_bias[f] + row_bias[b])      (bf16 operands and output)
 * What `(x @ W) + bias` is under bf16 autocast: the product a bf16 tensor, the bias an fp32 parameter, the sum cast to
 * bf16 by the next autocast op.  col_bias [F] / row_bias [B] nullable (row_bias serves the swapped-operand call that
 * writes a transposed projection).  d % 64 == 0.  Replaces Lorsa's q / k / v projections with their biases
 * (models/lorsa.py:784-829). */
int sae_encoder_gemm_bias(const void *x_bf16, const void *w_t_bf16, void *out_bf16, int64_t B, int64_t d, int64_t F,
                          const float *col_bias, const float *row_bias, void *stream);

/* The encoder product and the per-token TopK with the row read only where it matters.
 * sae_encoder_gemm_granule_max: sae_encoder_gemm for bf16 operands and bf16 output (F % 64 == 0) whose epilogue
 *   also writes granule_max [B, F / 64] (uint32): for every token and every aligned granule of 64 features the
 *   largest select key of the granule, the key of an element being the bit pattern of
 *   h1 = (bf16(pre) + b_enc) * scale when h1 > 0 and 0 otherwise (b_enc / scale nullable: 0 / 1).
 * sae_select_topk_row_granule: the result of sae_select_topk_row (same outputs, bit for bit) from pre and
 *   granule_max: the k-th largest granule maximum bounds the k-th largest key from below, so only the ~k granules
 *   that reach it are read from pre.  F % 64 == 0, F <= 262144, k <= 512; rows whose candidates do not fit the
 *   in-LDS list (mass ties) are redone from the whole row by a second launch of the general kernel.
 * n_groups > 1: that many independent products of one shape in one launch, every array stacked group after group
 *   (x [G, B, d], w_enc_t [G, F, d], pre [G, B, F], b_enc / scale [G, F], granule_max [G, B, F / 64]); the select
 *   then takes all G * B rows at once with rows_per_group = B (0: one group), so that row r uses the bias and scale
 *   of group r / B.
 * pre_rows (0: as many as rows): the groups may share ONE pre-activation matrix of pre_rows rows, row r then reading
 *   pre row r % pre_rows (a crosscoder: every head selects from the same summed encoding under its own decoder norms,
 *   models/crosscoder.py:353-382; the rows are then (head, token) and granule_max [n_heads * B, F / 64] comes from
 *   sae_granule_max with the same arguments).
 * Together they replace `hidden_pre = x @ W_E + b_E` followed by the TopK of `hidden_pre * decoder_norm`
 * (models/sae.py:324-341, utils/math.py:81-171). */
int sae_encoder_gemm_granule_max(const void *x_bf16, const void *w_enc_t_bf16, void *pre_bf16, int64_t n_groups, int64_t B,
                                 int64_t d, int64_t F, const float *b_enc, const float *scale, uint32_t *granule_max,
                                 void *stream);
int sae_select_topk_row_granule(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc, const float *scale,
                                int64_t B, int64_t F, int k, int64_t rows_per_group, int64_t pre_rows, int32_t *idx, float *val,
                                int64_t *row_off, int32_t *row_nnz, void *stream);
/* The two entry points above in the bf16 arithmetic of a dictionary held in bf16 (the keys of sae_select_topk_row_lowp:
 * the sum with the bias and the product with the scale each rounded to bf16; values rounded after the division). */
int sae_encoder_gemm_granule_max_lowp(const void *x_bf16, const void *w_enc_t_bf16, void *pre_bf16, int64_t n_groups, int64_t B,
                                      int64_t d, int64_t F, const float *b_enc, const float *scale, uint32_t *granule_max,
                                      void *stream);
int sae_select_topk_row_granule_lowp(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc, const float *scale,
                                     int64_t B, int64_t F, int k, int64_t rows_per_group, int64_t pre_rows, int32_t *idx,
                                     float *val, int64_t *row_off, int32_t *row_nnz, void *stream);

/* sae_select_topk_batch (bf16 pre, no feat_mask, F % 256 == 0) with the per-granule key maxima handed in
 * (granule_max [B, F / 64] of sae_encoder_gemm_granule_max for the same pre, b_enc, scale): the select's one pass over
 * the whole matrix shrinks to a histogram of the maxima; every later pass and the result are those of
 * sae_select_topk_batch.  Same workspace. */
int sae_select_topk_batch_granule(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc, const float *scale,
                                  int64_t B, int64_t F, int64_t k_total, const int64_t *k_total_dev, int32_t *idx, float *val,
                                  int64_t capacity, int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                                  int64_t workspace_bytes, void *stream);

/* sae_select_topk_batch for a dictionary whose dtype is bfloat16 (config.py:39), as sae_select_topk_row_lowp is to
 * sae_select_topk_row: pre is bf16, and the sum with the bias, the product with the scale and the final quotient are each
 * rounded to bf16, as the bf16 tensors around the reference's batch_topk closure are (models/sae.py:324-341,
 * models/sparse_dictionary.py:761-794).  b_enc / scale are fp32 copies of the bf16 bias / norms.  Many keys then share
 * the threshold's value; ties keep the lowest flattened indices b * F + f.  feat_mask as in sae_select_topk_row_lowp.
 * granule_max (or NULL): the maxima sae_encoder_gemm_granule_max_lowp left, as in sae_select_topk_batch_granule (no
 * feat_mask then, F a multiple of 256).  Same workspace. */
int sae_select_topk_batch_lowp(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc, const float *scale,
                               const float *feat_mask, int64_t B, int64_t F, int64_t k_total, const int64_t *k_total_dev,
                               int32_t *idx, float *val, int64_t capacity, int64_t *row_off, int32_t *row_nnz,
                               int64_t *total_out, void *workspace, int64_t workspace_bytes, void *stream);

/* granule_max [B, F / 64] of sae_encoder_gemm_granule_max for a bf16 pre that did not come out of that product
 * (Lorsa's head activations), or whose rows are shared by several groups of scales (a crosscoder's heads): one streaming
 * read per row.  rows_per_group and pre_rows as in sae_select_topk_row_granule (B counts the rows of granule_max). */
int sae_granule_max(const void *pre_bf16, const float *b_enc, const float *scale, int64_t B, int64_t F, int64_t rows_per_group,
                    int64_t pre_rows, uint32_t *granule_max, void *stream);

/* Per-layer codes -> one code over L * F features (the cross-layer transcoder's per-layer TopK, models/clt.py:232-387:
 * each layer keeps its own k, the decoders read all layers' entries of a token).  idx / val [L * B * k] and row_nnz
 * [L * B] are the outputs of one stacked select (row l * B + b: layer l, token b; slots row * k ..; ascending features).
 * out_idx / out_val [B * L * k], out_row_off / out_row_nnz [B]: token b's entries in slots b * L * k .., layer after
 * layer, feature ids l * F + f (ascending), unused slots zeroed; layer_cnt [B, L] = entries per (token, layer). */
int sae_merge_layer_codes(const int32_t *idx, const float *val, const int32_t *row_nnz, int64_t L, int64_t B, int64_t k,
                          int64_t F, int32_t *out_idx, float *out_val, int64_t *out_row_off, int32_t *out_row_nnz,
                          int32_t *layer_cnt, void *stream);

/* Codes of G groups over the same tokens and features -> one code holding every (token, feature) once (a crosscoder's
 * heads select from one summed encoding, models/crosscoder.py:246-305, so d loss / d pre[b, f] is the sum of the heads'
 * value gradients at (b, f) and the encoder's gradient rows need each pair once).  idx / val [G * B * k] and row_nnz
 * [G * B] are one stacked select's outputs (row g * B + b: group g, token b; slots row * k ..).  out_idx / out_val
 * [B * G * k], out_row_off / out_row_nnz [B]: token b's distinct features in slots b * G * k .., in order of first
 * appearance, each with the sum of its values over the token's rows (added in group order); unused slots zeroed.
 * G * k <= 1024. */
int sae_union_group_codes(const int32_t *idx, const float *val, const int32_t *row_nnz, int64_t G, int64_t B, int64_t k,
                          int32_t *out_idx, float *out_val, int64_t *out_row_off, int32_t *out_row_nnz, void *stream);

/* Batch-global TopK (BatchTopK): keep the k_total largest h1 > 0 over the whole [B, F] batch
 * (h0, h1 as above); ties at the threshold -> lowest flattened index b * F + f.  If fewer than
 * k_total entries are positive, all positives are kept.
 *   feat_mask (nullable, fp32 0/1 [F]): the aux-k form, h1 = ((h0 * scale) / scale) * feat_mask * scale,
 *     i.e. `hidden_pre * is_dead * decoder_norm` op for op;
 *   k_total_dev (nullable): read k_total from device memory instead (k' * B with k' known only there);
 *   idx/val have room for `capacity` entries (entries beyond it are dropped; k_total is the
 *     natural capacity); row_off/row_nnz [B] describe the variable-length rows; total_out
 *     (nullable, device int64) receives the number of kept entries.
 * workspace: sae_select_topk_batch_workspace_bytes(B, F) bytes, 256-byte aligned: about B * F / 4 bytes
 *   (one largest key per 32 elements, and a candidate list of B * F / 64 + 1024 keys with their features);
 *   F <= 2^30.
 * Replaces the batchtopk closure (models/sparse_dictionary.py:761-794) + utils/math.py:81-171
 * with dim=(-2,-1), and the dead-latent select of the aux-k loss (sparse_dictionary.py:952-972). */
int64_t sae_select_topk_batch_workspace_bytes(int64_t B, int64_t F);
int sae_select_topk_batch(const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                          const float *feat_mask, int64_t B, int64_t F, int64_t k_total,
                          const int64_t *k_total_dev, int32_t *idx, float *val, int64_t capacity,
                          int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                          int64_t workspace_bytes, void *stream);

/* ---- sparse decoder --------------------------------------------------------------- */

/* recon[b, :] = sum_s val[s] * W_D[idx[s], :] + b_dec,  s over token b's slots.
 * w_dec [F, d] in w_dtype (bf16 shadow or fp32 master); recon [B, d] fp32; b_dec fp32 [d]
 * or null.  Requires d % 8 == 0.
 * Replaces `feature_acts @ self.W_D + self.b_D` (models/sae.py:367-371) and the Triton SpMM
 * (kernels/kernels.py:382-436). */
int sae_sparse_decode_fwd(const int32_t *idx, const float *val, const int64_t *row_off,
                          const int32_t *row_nnz, const void *w_dec, int w_dtype, const float *b_dec,
                          float *recon, int64_t B, int64_t d, int64_t F, void *stream);

/* dval[s] = grad_recon[b, :] . W_D[idx[s], :] for every valid slot s of token b
 * (0 for unused slots).  Replaces the "dense x dense -> sparse out" backward
 * (kernels/kernels.py:326-379, 562-563). */
int sae_sparse_decode_bwd_dval(const int32_t *idx, const int64_t *row_off, const int32_t *row_nnz,
                               const float *grad_recon, const void *w_dec, int w_dtype, float *dval,
                               int64_t B, int64_t d, int64_t F, int64_t n_slots, void *stream);

/* Fused forward+backward of decode and the reconstruction loss for one batch:
 *   recon = decode(idx, val) + b_dec
 *   loss_tok[b]     = tok_w[b] * sum_j (recon[b,j] - label[b,j])^2
 *   grad_recon[b,:] = 2 * tok_w[b] * (recon[b,:] - label[b,:])
 *   dval[s]         = grad_recon[b,:] . W_D[idx[s],:]
 * tok_w[b] is the per-token weight of the masked mean (mask[b] / mask.sum(); 1/B without a
 * mask), or null for 1.  recon may be null when the caller does not need it.
 * Replaces models/sae.py:367-371 + models/sparse_dictionary.py:881-886
 * (+ utils/tensor_specs.py:64-84) and their autograd twins. */
int sae_sparse_decode_mse_fused(const int32_t *idx, const float *val, const int64_t *row_off,
                                const int32_t *row_nnz, const void *w_dec, int w_dtype,
                                const float *b_dec, const float *label, const float *tok_w,
                                float *recon, float *loss_tok, float *grad_recon, float *dval,
                                int64_t B, int64_t d, int64_t F, int64_t n_slots, void *stream);

/* sae_sparse_decode_mse_fused for a code that several decoders share (the cross-layer transcoder's prefix decodes,
 * models/clt.py:630-709): the value gradients are ADDED to dval_acc [n_slots] (slots a call does not visit keep their
 * value; the caller clears the array before the first call), so that the sum over the decoders needs no pass of its own.
 * Each slot is written by the one wave that owns its token: no atomics, the additions happen in call order. */
int sae_sparse_decode_mse_fused_acc(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz,
                                    const void *w_dec, int w_dtype, const float *b_dec, const float *label, const float *tok_w,
                                    float *recon, float *loss_tok, float *grad_recon, float *dval_acc, int64_t B, int64_t d,
                                    int64_t F, int64_t n_slots, void *stream);

/* ---- sparse backward -------------------------------------------------------------- */

/* Feature-major index of a sparse code (a CSR transpose): for every feature f the list of
 * slots s with idx[s] == f, in ascending slot (= token) order.
 *   feat_ptr  int32 [F + 1]   segment bounds,
 *   feat_slot int32 [n_valid] slot ids grouped by feature (n_valid = sum row_nnz),
 *   slot_tok  int32 [n_slots] token of every slot (filled for valid slots).
 * workspace: sae_feature_index_workspace_bytes(B, F, n_slots) bytes.
 * Replaces the global sort into COO (kernels/kernels.py:61-134). */
int64_t sae_feature_index_workspace_bytes(int64_t B, int64_t F, int64_t n_slots);
int sae_build_feature_index(const int32_t *idx, const int64_t *row_off, const int32_t *row_nnz,
                            int64_t B, int64_t F, int64_t n_slots, int32_t *feat_ptr,
                            int32_t *feat_slot, int32_t *slot_tok, void *workspace,
                            int64_t workspace_bytes, void *stream);

/* out[f, :] = sum_{s in segment f} coef[s] * dense[slot_tok[s], :]   for every f in [0, F)
 * (rows with an empty segment are written as zeros, so `out` needs no prior clearing);
 * optionally bias_out[f] = sum coef[s].  dense [B, d] in dense_dtype, out [F, d] fp32.
 * With coef = val and dense = grad_recon this is dW_D; with coef = d(pre) and dense = x it
 * is dW_E^T and bias_out = db_E.
 * Replaces the sorted atomic-add SpMM (kernels/kernels.py:137-225) and the dense
 * `f^T @ grad` / `x^T @ dh` GEMMs autograd runs. */
int sae_sparse_grad_rows(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                         const float *coef, const void *dense, int dense_dtype, float *out,
                         float *bias_out, int64_t F, int64_t d, void *stream);

/* ---- optimiser -------------------------------------------------------------------- */

/* One bias-corrected Adam update over n contiguous fp32 elements (p, m, v in/out):
 *   m = b1*m + (1-b1)*g;  v = b2*v + (1-b2)*g*g;
 *   p -= lr / (1 - b1^t) * m / (sqrt(v) / sqrt(1 - b2^t) + eps)
 * (torch.optim.Adam, no weight decay, no amsgrad: trainer.py:375-390).  step = t >= 1.
 * g is fp32 or bf16 (g_dtype): the weight gradient of an autocast matmul is a bf16 tensor that the framework
 * widens to fp32 in a pass of its own before torch.optim.Adam reads it; here it is widened as it is read.
 * shadow_bf16 (nullable) receives bf16(p) for the next step's GEMM / gather operands.
 * row_norm_out (nullable, requires row_len > 0 and n % row_len == 0) receives the L2 norm
 * of every updated row of length row_len, i.e. the next step's decoder_norm().
 * row_grad_coef (nullable, fp32 [n / row_len], same requirement on row_len): the gradient of row r is
 * g + row_grad_coef[r] * p.  This is how the gradient that reaches W_D through decoder_norm()
 * (models/sae.py:136-147: d W_D[f, :] += (d n_f / n_f) W_D[f, :], e.g. from the tanh sparsity penalty,
 * models/sparse_dictionary.py:897-906) is applied without a pass over [F, d] of its own. */
int sae_adam_step(float *p, const void *g, int g_dtype, float *m, float *v, int64_t n, double lr, double beta1,
                  double beta2, double eps, int64_t step, void *shadow_bf16, float *row_norm_out,
                  int64_t row_len, const float *row_grad_coef, void *stream);

/* Adam on a feature-major weight matrix [F, d] whose gradient is given in factored form:
 *   g[f, :] = sum_{s in segment f of the feature index} coef[s] * dense[slot_tok[s], :]
 * (the quantity sae_sparse_grad_rows would write).  The row gradient is formed in registers and
 * consumed at once; no dense gradient is stored.  Same update rule, scalars and by-products
 * (shadow_bf16, row_norm_out) as sae_adam_step; bias_grad_out (nullable) receives
 * sum_{s in segment f} coef[s], the gradient of the per-feature bias.  Bit-identical to
 * sae_sparse_grad_rows followed by sae_adam_step.  grad_scale (nullable): device float[1]; the
 * row gradient and bias_grad_out are multiplied by it before use, which is clip_grad_norm's
 * `grad.mul_(factor)` (optim.py:280-292) with the factor left on the device.
 * grad_sq_nnz_acc (nullable): device double[2]; sum g^2 and #(g != 0) of the gradient this call consumes are
 * added to it (the sums of sae_sparse_rows_grad_sq_nnz, as a by-product: the every-step gradient-norm
 * diagnostic of trainer.py:629-639 then costs no pass of its own).  It needs `workspace`, device memory of
 * sae_sparse_rows_grad_sq_nnz_workspace_bytes(F) bytes, 16-byte aligned; both may be NULL / 0 otherwise.
 * extra_map / extra_rows / extra_bias (nullable, the first two together): a block of gradient rows held densely,
 * for features whose gradient is not worth factoring (the aux-k loss touches every dead feature from a large
 * share of the tokens; its rows come from three small GEMMs).  extra_map: device int32[F], -1 or the row of
 * extra_rows ([n, d] fp32, 16-byte aligned) that is added to feature f's gradient; extra_bias: fp32[n] added to
 * bias_grad_out likewise.
 * row_grad_coef (nullable, fp32 [F]): as in sae_adam_step, the gradient of row f is g + row_grad_coef[f] * p[f, :] (product
 * and sum rounded separately): the gradient that reaches W_D through decoder_norm().
 * Replaces loss.backward()'s dense `f^T @ grad` / `x^T @ dh` GEMMs together with
 * torch.optim.Adam.step for W_D / W_E (trainer.py:627-647). */
int sae_adam_step_sparse_rows(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                              const float *coef, const void *dense, int dense_dtype, float *p, float *m,
                              float *v, int64_t F, int64_t d, double lr, double beta1, double beta2,
                              double eps, int64_t step, void *shadow_bf16, float *row_norm_out,
                              float *bias_grad_out, const float *grad_scale, double *grad_sq_nnz_acc,
                              void *workspace, int64_t workspace_bytes, const int32_t *extra_map,
                              const float *extra_rows, const float *extra_bias, const float *row_grad_coef, void *stream);

/* The two Adam entry points above for a dictionary whose dtype is bfloat16 (config.py:39 `dtype`; parameters,
 * gradients and both moments are then bf16 tensors and torch.optim.Adam, trainer.py:375-390, updates them with its
 * multi-tensor element-wise operations): p_bf16, m_bf16, v_bf16 are bf16 arrays, there is no shadow copy (the
 * parameter is its own bf16 operand), and the update rounds to bf16 after every element-wise operation torch
 * performs -- the gradient itself; lerp for m; mul, then addcmul for v; sqrt, the division by sqrt(1 - beta2^t)
 * and the addition of eps for the denominator; addcdiv for p.  row_norm_out is the fp32 norm of the updated bf16
 * rows.  extra_map / extra_rows / extra_bias as in sae_adam_step_sparse_rows (fp32 rows, added before the gradient is
 * rounded to bf16). */
int sae_adam_step_lowp(void *p_bf16, const void *g, int g_dtype, void *m_bf16, void *v_bf16, int64_t n, double lr,
                       double beta1, double beta2, double eps, int64_t step, float *row_norm_out, int64_t row_len,
                       const float *row_grad_coef, void *stream);
int sae_adam_step_sparse_rows_lowp(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                   const float *coef, const void *dense, int dense_dtype, void *p_bf16, void *m_bf16,
                                   void *v_bf16, int64_t F, int64_t d, double lr, double beta1, double beta2,
                                   double eps, int64_t step, float *row_norm_out, float *bias_grad_out,
                                   const float *grad_scale, double *grad_sq_nnz_acc, void *workspace,
                                   int64_t workspace_bytes, const int32_t *extra_map, const float *extra_rows,
                                   const float *extra_bias, void *stream);

/* SparseAdam (optim.py:142-254) over n contiguous fp32 elements: m *= b1, v *= b2 everywhere;
 * where g != 0 also m += (1-b1) g, v += (1-b2) g^2 and
 *   p -= lr * sqrt(1 - b2^t) / (1 - b1^t) * m / (sqrt(v) + eps);
 * a gradient that is zero everywhere leaves p, m, v and the step counter untouched.
 * step_state: device float[1], the number of steps taken so far (in/out; t = step_state + 1);
 * flag_workspace: device int32[1] scratch.  No host synchronisation (the reference's
 * `if not grad.any(): continue` is evaluated on the device). */
int sae_sparse_adam_step(float *p, const float *g, float *m, float *v, int64_t n, double lr, double beta1,
                         double beta2, double eps, float *step_state, int32_t *flag_workspace,
                         void *shadow_bf16, void *stream);

/* acc[0] += sum_i g[i]^2, acc[1] += #{i : g[i] != 0}, both accumulated in fp64 (acc: device double[2],
 * cleared by the caller before the first tensor).  The two quantities behind
 * compute_grad_norm (optim.py:257-277): ||g|| / sqrt(#non-zero). */
int sae_grad_sq_nnz(const float *g, int64_t n, double *acc, void *stream);

int64_t sae_sparse_rows_grad_sq_nnz_workspace_bytes(int64_t F);

/* The same two sums for a weight gradient held in factored form (see sae_adam_step_sparse_rows): every
 * feature's row is rebuilt in registers and reduced, the dense gradient is never stored.  This is what
 * the trainer's every-step clip_grad_norm / grad-norm diagnostic (trainer.py:629-639, optim.py:257-292)
 * needs from W_E and W_D.  acc as in sae_grad_sq_nnz (accumulated into, in a fixed order);
 * bias_grad_out (nullable) receives sum_{s in segment f} coef[s]; workspace: device memory of
 * sae_sparse_rows_grad_sq_nnz_workspace_bytes(F) bytes, 16-byte aligned; extra_map / extra_rows / extra_bias as in
 * sae_adam_step_sparse_rows. */
int sae_sparse_rows_grad_sq_nnz(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                const float *coef, const void *dense, int dense_dtype, int64_t F, int64_t d,
                                double *acc, float *bias_grad_out, void *workspace, int64_t workspace_bytes,
                                const int32_t *extra_map, const float *extra_rows, const float *extra_bias,
                                void *stream);

/* Reconstruction loss, aux-k loss and the two output gradients of a step whose aux reconstruction is dense, one
 * pass over [B, d] (d a multiple of 4, 16-byte aligned rows):
 *   rec_tok[b] = w_b sum_j (recon - label)^2                      (l_rec = sum_b rec_tok, w_b = tok_w[b] or 1)
 *   aux_tok[b] = w_b sum_j ((label - recon) - aux_recon)^2        (l_aux = alpha sum_b aux_tok)
 *   g_aux      = (-2 alpha w_b) ((label - recon) - aux_recon)     = d loss / d aux_recon
 *   grad_recon = (2 w_b) (recon - label) + g_aux                  = d loss / d recon (the residual carries gradient)
 * aux_recon may be null (no dead feature: aux_tok and g_aux are then not written and grad_recon is the first term);
 * grad_recon_bf16 (nullable) receives grad_recon rounded to bf16.
 * Replaces models/sparse_dictionary.py:871-886 (l_rec) and :973-991 (the aux-k residual loss) with their autograd twins. */
int sae_mse_auxk_fused(const float *recon, const float *label, const float *aux_recon, const float *tok_w, double alpha,
                       int64_t B, int64_t d, float *rec_tok, float *aux_tok, float *g_aux, float *grad_recon,
                       void *grad_recon_bf16, void *stream);

/* [rows, cols] fp32 or bf16 -> bf16 [cols, rows] (round to nearest even).
 *   mask (nullable, fp32 [rows, cols]): entries whose mask is not positive are written as 0;
 *   col_part (nullable, fp32 [ceil(rows / 64), cols]): per 64-row tile, the column sums of the (masked) fp32
 *     values, in a fixed order; summing its rows (sae_col_sum) gives the column sums of the masked matrix.
 * The operands autograd transposes inside the backward of the aux-k products (`aux_acts @ W_D` and the encoder
 * product over the dead features, models/sparse_dictionary.py:952-991): A^T, G^T, x^T for dW = A^T G, and
 * d pre^T = (dA masked to the kept entries)^T with its column sums = the dead features' bias gradient. */
int sae_transpose_to_bf16(const void *src, int src_dtype, const float *mask, int64_t rows, int64_t cols, void *dst,
                          float *col_part, void *stream);

/* Sparse code -> dense [B, n_cols] rows, in fp32 and / or bf16 (either pointer may be null, not both): token b's
 * entries idx/val[row_off[b] .. row_off[b] + row_nnz[b]) at their columns, zeros elsewhere; indices outside
 * [0, n_cols) are dropped.  A token's indices must be distinct.
 * The reference's TopK / BatchTopK activation returns this dense matrix (utils/math.py:81-171 scatter); here it is
 * wanted only for the compact block of dead features of the aux-k term (models/sparse_dictionary.py:952-972). */
int sae_code_to_dense(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz, int64_t B,
                      int64_t n_cols, float *dense_f32, void *dense_bf16, void *stream);

/* The same matrix transposed and in bf16: dense_t_bf16 [n_cols, B] (cleared, then token b's entries written down column
 * b).  The left operand of a dense weight-gradient product over the token axis, dW_D = acts^T grad_recon: what autograd
 * forms for `feature_acts @ W_O` (models/lorsa.py:765-782), and cheaper than gathered gradient rows when the dictionary
 * is small against the batch (d_sae / k below a few hundred). */
int sae_code_to_dense_t(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz, int64_t B,
                        int64_t n_cols, void *dense_t_bf16, void *stream);

/* ---- Dense feature activations -> sparse code ----------------------------------------------------------------
 * The conversion in front of the sparse decoder kernels when a caller hands over a dense [B, F] activation matrix
 * (fp32 or bf16): get_sparse_representation (kernels/kernels.py:14-58: nonzero, bincount, cumsum, scatter into a padded
 * [B, nnz_max] pair) as two passes.
 *   sae_dense_row_nnz: row_nnz[b] = #{f : dense[b, f] != 0}.
 *   sae_dense_to_code: given row_off (int64 [B], e.g. the exclusive prefix sum of row_nnz), token b's non-zero entries
 *     are written in ascending feature order to idx / val [capacity] from slot row_off[b] on; entries that would land at
 *     or past `capacity` are dropped, and `row_nnz` (nullable, int32 [B], rewritten) is cut to the number of entries that
 *     were written for each token, so that a code with an undersized capacity stays walkable (truncated, never out of
 *     bounds).  (row_off, row_nnz, idx, val) is then a sparse code as the select entry points emit it. */
int sae_dense_row_nnz(const void *dense, int dtype, int64_t B, int64_t F, int32_t *row_nnz, void *stream);
int sae_dense_to_code(const void *dense, int dtype, int64_t B, int64_t F, const int64_t *row_off, int32_t *idx, float *val,
                      int64_t capacity, int32_t *row_nnz, void *stream);

/* ---- Activation batches from a shuffle buffer -----------------------------------------------------------
 * dst[i, :] = cast(scale * src[row_idx[i], :]) for i < n_rows: one batch drawn from a token buffer that
 * stays where it is in HBM.  Replaces ActivationBuffer.shuffle / yield_batch
 * (activation/processors/activation.py:96-164), which permute and re-concatenate the whole buffer for every
 * refill and every batch; here a shuffle permutes indices only and a batch is this one gather, with the
 * dtype override (activation/processors/activation.py:397-410) and a normalisation factor folded in.
 * src: [n_src_rows, d], dst: [n_rows, d], SAE_F32 or SAE_BF16 each; row_idx: device int64[n_rows], every
 * entry in [0, n_src_rows) (an entry outside leaves its output row untouched). */
int sae_gather_rows(const void *src, int src_dtype, const int64_t *row_idx, int64_t n_src_rows, int64_t n_rows,
                    int64_t d, void *dst, int dst_dtype, double scale, void *stream);

/* ---- Training metrics from the sparse code ----------------------------------------------------------
 * The per-step quantities behind FrequencyMetric, MeanFeatureActMetric and L0Metric (metrics.py:102-127,
 * 189-204, 258-288), which the reference computes from the dense [B, F] feature_acts:
 *   freq_acc[f] += sum_b w_b [acts[b, f] > 0]        (act_freq_scores; w_b = tok_w[b], 1 when tok_w is NULL)
 *   l0_tok[b]    = #{f : acts[b, f] > 0}             (nullable)
 *   totals[0]   += sum of all kept values            (feature_acts.sum())
 *   totals[1]   += #{(b, f) : acts[b, f] > 0}        (feature_acts.gt(0).sum(), unmasked as in the reference)
 *   totals[2]   += sum_b w_b l0_tok[b]               (the masked L0 sum)
 * idx / val / row_off / row_nnz: a sparse code as the select kernels emit it.  freq_acc (float[F], nullable)
 * and totals (double[3], nullable) are accumulated into, so a running sum over steps needs no extra pass. */
int sae_code_stats(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz,
                   const float *tok_w, int64_t B, int64_t F, float *freq_acc, float *l0_tok, double *totals,
                   void *stream);

/* ExplainedVarianceMetric and L2NormErrorMetric (metrics.py:207-255, 291-314) from label / recon [B, d] fp32 and the
 * (masked) column mean of label:  with se_b = |recon_b - label_b|^2, var_b = |label_b - mean|^2 and
 * <.> = sum_b w_b (.) / sum_b w_b,
 *   acc[0] += 1 - <se> / <var>         explained_variance
 *   acc[1] += <1 - se / var>           explained_variance_legacy
 *   acc[2] += <sqrt(se)>               l2_norm_error
 *   acc[3] += <sqrt(se)> / <|label|>   l2_norm_error_ratio
 * acc: device double[4], accumulated into; step_out (nullable): device float[4], this step's values;
 * tok_workspace: device float[3 B]. */
int sae_recon_stats(const float *label, const float *recon, const float *label_mean, const float *tok_w,
                    int64_t B, int64_t d, float *tok_workspace, double *acc, float *step_out, void *stream);

/* ---- JumpReLU with straight-through threshold gradient --------------------------------------------
 * Replaces STEFunction / JumpReLU (activation_functions.py:15-140) as the SAE encoder applies it
 * (models/sae.py:136-160: scale by the decoder norm, activate, unscale) together with the sparsity
 * terms that read the same [B, F] data: the tanh penalty (models/sparse_dictionary.py:893-894) and the
 * Lp penalty (models/sparse_dictionary.py:927-938).
 * With h = pre + b_enc, s = scale[f] (1 when scale is NULL), u = h * s, n = pen_norm[f] (1 when NULL;
 * the decoder norm the penalties weigh by, whether or not the activation is scaled by it):
 *   acts[b, f]   = u > theta[f] ? u / s : 0                       (dtype of `pre`)
 *   tanh_tok[b]  = sum_f tanh(tanh_c * acts * n)                  (optional)
 *   lp_tok[b]    = sum_f relu(theta - h) * n                      (optional)
 *   l0_tok[b]    = number of kept features                        (optional)
 * pre, acts: [B, F] row-major, SAE_F32 or SAE_BF16; F must be a multiple of 8. */
int sae_jumprelu_fwd(const void *pre, int dtype, const float *b_enc, const float *scale, const float *pen_norm,
                     const float *theta, int64_t B, int64_t F, double tanh_c, void *acts, float *tanh_tok, float *lp_tok, float *l0_tok,
                     void *stream);

int64_t sae_jumprelu_bwd_workspace_bytes(int64_t B, int64_t F);

/* Backward of the above.  d_acts [B, F] is the gradient arriving at acts; g_tanh [B] / g_lp [B] are the
 * gradients arriving at tanh_tok / lp_tok (NULL when that term is unused).  With
 * ga = d_acts + g_tanh[b] * tanh_c * n * (1 - tanh^2):
 *   d_pre[b, f]  = (u > theta ? ga : 0) - (theta > h ? g_lp[b] * n : 0)
 *   d_bias[f]    = sum_b d_pre
 *   d_theta[f]   = sum_b [ |u - theta| < window / 2 and u > 0 ] * (ga / s) * (-theta / window)  +  sum_b [theta > h] g_lp[b] n
 *                  (the rectangle-window estimator of activation_functions.py:45-61; the gradient of
 *                  log theta is d_theta * theta)
 *   d_pen_norm[f] = sum_b g_tanh[b] tanh_c acts (1 - tanh^2) + sum_b g_lp[b] relu(theta - h)     (optional;
 *                  the derivative terms of acts with respect to `scale` cancel, so `scale` gets no gradient)
 * The per-feature sums are reduced in a fixed order (deterministic). */
int sae_jumprelu_bwd(const void *pre, int dtype, const float *b_enc, const float *scale, const float *pen_norm,
                     const float *theta, const void *d_acts, const float *g_tanh, double tanh_c, const float *g_lp, double window,
                     int64_t B, int64_t F, void *d_pre, float *d_bias, float *d_theta, float *d_pen_norm,
                     void *workspace, int64_t workspace_bytes, void *stream);

/* ---- Causal attention with grouped value heads (low-rank sparse attention) -------------------------------
 * Replaces F.scaled_dot_product_attention(query, key, value, scale, is_causal=True) as LowRankSparseAttention calls it
 * (models/lorsa.py:650-660, 714-724) and its autograd backward: n_heads query/key heads of width d_qk, and per head a
 * value of width d_v whose columns are the d_v rank-1 value heads (dictionary features) that share the head's pattern.
 *   out[b, s, h, :] = sum_{s' <= s} softmax_{s'}(scale * q[b, s, h, :] . k[b, s', h, :]) * v[b, s', h, :]
 * bf16 operands, fp32 accumulation, probabilities rounded to bf16 before they multiply the values (as the library's
 * fused kernels do).  T = n_batch * seq, token t = b * seq + s.  Layouts: "natural" [T, n_heads * width] (heads side by
 * side: what x @ W gives) and "transposed" [n_heads * width, T].
 *   q, k      [T, n_heads * d_qk];  v [T, n_heads * d_v]   (natural: a product over positions reads its operand across
 *             the rows of the LDS tile with transposing reads, so no transposed copies are taken)
 *   out       [T, n_heads * d_v] bf16;  lse fp32 [n_batch, n_heads, seq] = log sum_{s'} exp(scale * q . k)
 * Requires d_qk in {32, 64}, d_v in {32, 64, 128}, seq % 8 == 0, at most 2^24 tokens.  Projection biases belong in the
 * products that form q, k, v (sae_encoder_gemm_bias). */
int sae_attention_fwd(const void *q, const void *k, const void *v, int64_t n_batch, int64_t seq, int64_t n_heads, int64_t d_qk,
                      int64_t d_v, double scale, void *out, float *lse, void *stream);

/* Backward of sae_attention_fwd.  q, k, v, out, dout natural; lse from the forward pass; workspace: device
 * float[2 * n_batch * n_heads * seq] (D = rowsum(dout * out), and the log-sum-exp in the log2 domain).  Outputs, bf16,
 * TRANSPOSED: dqt, dkt [n_heads * d_qk, T], dvt [n_heads * d_v, T], the layout in which they are the left operand of the
 * weight-gradient product over the token axis (a projection bias's gradient is the row sum, sae_row_sum).  No atomics:
 * reproducible. */
int sae_attention_bwd(const void *q, const void *k, const void *v, const void *out, const void *dout, const float *lse,
                      int64_t n_batch, int64_t seq, int64_t n_heads, int64_t d_qk, int64_t d_v, double scale, float *workspace,
                      void *dqt, void *dkt, void *dvt, void *stream);

/* Rotary positional embedding of Lorsa's queries / keys between projection and scores (models/lorsa.py:821-824, 864-904;
 * tables as models/lorsa.py:525-575 builds them, cos / sin fp32 [n_ctx, rotary_dim]).  acc fp32 [T, n_heads d_head] holds
 * the projection's accumulators, T = batches x seq tokens, a token's position is its index inside its sequence;
 *   out = bf16(rotate(float(bf16(acc)) + bias)),
 * i.e. the bf16 product plus the fp32 bias, rotated in fp32 and rounded once, as the reference's tensors are under bf16
 * autocast.  The first rotary_dim elements of a head are rotated in pairs (adjacent_pairs: (2i, 2i+1), else
 * (j, j + rotary_dim / 2)), the rest pass through.  rotary_dim a multiple of 16, d_head and seq multiples of 8. */
int sae_rotary_fwd(const float *acc, const float *bias, const float *cos_tab, const float *sin_tab, int64_t n_ctx, int64_t T,
                   int64_t seq, int64_t n_heads, int64_t d_head, int64_t rotary_dim, int adjacent_pairs, void *out_bf16,
                   void *stream);
/* The transpose of that rotation, in place on a gradient held transposed, grad_t bf16 [n_heads d_head, T] (what
 * sae_attention_bwd leaves for queries and keys): rows in pairs, dx[a] = dy[a] cos[a] + dy[b] sin[b],
 * dx[b] = dy[b] cos[b] - dy[a] sin[a], rounded to bf16.  cos_t / sin_t are the tables transposed, fp32 [rotary_dim, n_ctx]. */
int sae_rotary_bwd_t(void *grad_t_bf16, const float *cos_t, const float *sin_t, int64_t n_ctx, int64_t T, int64_t seq,
                     int64_t n_heads, int64_t d_head, int64_t rotary_dim, int adjacent_pairs, void *stream);

/* out[r] = sum_c src[r, c] (fp32 sum, fixed order) for src [rows, cols] fp32 or bf16.  The bias gradients autograd forms by
 * summing over tokens, for gradients held transposed ([features, tokens]). */
int sae_row_sum(const void *src, int src_dtype, int64_t rows, int64_t cols, float *out, void *stream);

/* The sparse form of the JumpReLU step, for dictionaries whose activations have become sparse (what the reference
 * reaches for with its sparsity gate, models/sae.py:355-367, and the sparsity-gated backward of
 * kernels/kernels.py:475-539): instead of a dense [B, F] activation, a sparse code of every token's kept features
 * (u > theta: value u / s, in_window as below) and of the features inside the straight-through window that are not kept
 * (|u - theta| < window / 2 and u > 0: value 0, in_window 1), with h, s, u, n as for sae_jumprelu_fwd.
 *   sae_jumprelu_select_count: row_nnz[b] = number of such entries of token b.
 *   sae_jumprelu_select_emit:  given row_off (int64 [B], the exclusive prefix sum of row_nnz), writes token b's entries in
 *     ascending feature order to idx / val / in_window [capacity] from slot row_off[b] on (entries at or past `capacity`
 *     are dropped), and per token tanh_tok[b] = sum over kept features of tanh(tanh_c * value * n) and l0_tok[b] = number
 *     of kept features (both nullable).
 * (row_off, row_nnz, idx, val) is a sparse code as the TopK select emits it: sae_sparse_decode_mse_fused gives the value
 * gradients of all entries (the flagged ones included: their threshold gradient needs them), sae_build_feature_index and
 * the factored optimizer pass take it as it is.  F must be a multiple of 8.
 * granule_margin (nullable; fp32 [B, F / 64], F % 64 == 0, F <= 262144): the second output of
 * sae_encoder_gemm_jumprelu_margin for the same pre, b_enc, scale and theta.  Only granules whose margin reaches
 * -window / 2 are then read from pre; the entries are the same (the per-token tanh sums add their terms in another order). */
int sae_jumprelu_select_count(const void *pre, int dtype, const float *b_enc, const float *scale, const float *theta,
                              const float *granule_margin, double window, int64_t B, int64_t F, int32_t *row_nnz, void *stream);
int sae_jumprelu_select_emit(const void *pre, int dtype, const float *b_enc, const float *scale, const float *pen_norm,
                             const float *theta, const float *granule_margin, double window, double tanh_c, int64_t B, int64_t F,
                             const int64_t *row_off, int32_t *idx, float *val, float *in_window, int64_t capacity, float *tanh_tok,
                             float *l0_tok, void *stream);

/* sae_encoder_gemm (bf16 operands and output, d % 64 == 0, F % 64 == 0) whose epilogue also writes
 * granule_margin [B, F / 64] (fp32): for every token and aligned granule of 64 features the largest
 * (bf16(pre) + b_enc) * scale - theta, product and difference rounded separately as in the activation kernels
 * (b_enc / scale nullable: 0 / 1).  Replaces `x @ W_E` ahead of the sparse JumpReLU select (models/sae.py:323-324). */
int sae_encoder_gemm_jumprelu_margin(const void *x_bf16, const void *w_enc_t_bf16, void *pre_bf16, int64_t B, int64_t d, int64_t F,
                                     const float *b_enc, const float *scale, const float *theta, float *granule_margin,
                                     void *stream);

/* out_a[f] = sum over the slots of feature f (feat_ptr / feat_slot of sae_build_feature_index) of a[slot], and the same
 * for b -> out_b (b, out_b nullable): the per-feature sums autograd forms by summing a dense [B, F] gradient over the
 * tokens (threshold and decoder-norm gradients of the sparse JumpReLU step), in a fixed order. */
int sae_feature_segment_sums(const int32_t *feat_ptr, const int32_t *feat_slot, const float *a, const float *b, int64_t F,
                             float *out_a, float *out_b, void *stream);

/* Measurement aid, no counterpart in the reference: n_workgroups x 4 waves each issue iters x 32
 * v_mfma_f32_16x16x32_bf16 from registers (no memory traffic in the loop) and write one float per lane to
 * out [n_workgroups * 256].  *flop_out (host, optional) receives the flop count of the launch.  The rate it
 * reaches is the matrix cores' ceiling on the card at the clock it runs at, which sae_encoder_gemm is read against. */
int sae_mfma_probe(float *out, int64_t n_workgroups, int64_t iters, double *flop_out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SAE_HIP_H */

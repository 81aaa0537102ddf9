/*
 * tlce.h — C ABI of the MI355X (gfx950) fused linear cross-entropy library
 * (libtlce_gfx950.so).
 *
 * The library replaces the device half of the reference's
 * `dllm_fused_linear_ce_v3` extension for the LM-head projection +
 * masked-token cross-entropy (forward and backward).  Every entry point takes
 * raw device pointers, sizes and a HIP stream; nothing here allocates, frees or
 * synchronises: the caller owns outputs and workspaces and sizes them with the
 * `*_workspace_bytes` helpers.  All matrices are contiguous row-major.
 *
 * Reference interfaces replaced (paths relative to the reference tree):
 *   chunked_linear_ce_forward               dllm_parallel/core/csrc/fused_linear_ce/fused_linear_ce.cpp:94-123
 *   chunked_linear_ce_backward              dllm_parallel/core/csrc/fused_linear_ce/fused_linear_ce.cpp:125-162
 *   chunked_linear_ce_backward_frozen_weight dllm_parallel/core/csrc/fused_linear_ce/fused_linear_ce.cpp:164-207
 *   (their device side: fused_linear_ce_cuda.cu:898-989 and :991-1172)
 *   row compaction at the loss call sites   dllm_parallel/core/models/backbones/nemotron/model.py:4234-4253
 *
 * Conventions
 *   - every function returning `int` returns 0 on success, non-zero on failure;
 *     `tlce_last_error()` then holds a thread-local message.
 *   - `stream` is a `hipStream_t` passed as `void*` (NULL = the null stream).
 *   - `dtype` is one of TLCE_DTYPE_*; hidden, weight and gradients share it.
 *   - `bias` is always float32 (the reference converts it the same way,
 *     fused_linear_ce_cuda.cu:913-916); NULL means "no bias".
 *   - `row_idx` (int64, ascending, length m) maps compacted row r to its
 *     position in the un-compacted [n_out] token axis; NULL means rows are
 *     already in place (n_out == m).
 *   - `exclude_index < 0` means no excluded vocabulary column;
 *     `logit_softcap <= 0` means no soft cap.
 */
#ifndef TLCE_H_
#define TLCE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TLCE_VERSION 1

enum {
  TLCE_DTYPE_F32 = 0,
  TLCE_DTYPE_F16 = 1,
  TLCE_DTYPE_BF16 = 2
};

/* reduction codes, same numbering as the reference binding shim
 * (dllm_parallel/core/kernels/chunked_linear_ce_native.py:366-373) */
enum {
  TLCE_REDUCTION_NONE = 0,
  TLCE_REDUCTION_SUM = 1,
  TLCE_REDUCTION_MEAN = 2
};

/* Library version (TLCE_VERSION it was built with). */
int tlce_version(void);

/* Thread-local text of the last failure on the calling thread ("" if none). */
const char* tlce_last_error(void);

/* 0 when `device` is a gfx950 GPU this library was compiled for.  Replaces
 * the architecture check of the reference's packaged-kernel loader
 * (dllm_parallel/core/kernels/runtime.py:189-387). */
int tlce_check_device(int device);

/* ---- masked-position compaction / gather --------------------------------
 * Device counterpart of `_compact_valid_loss_rows`
 * (nemotron/model.py:4234-4253): row_idx = nonzero(labels != ignore_index),
 * ascending int64, then index_select of the loss-bearing rows. */

/* Bytes of scratch `tlce_compact_rows` needs for `n` labels. */
int64_t tlce_compact_workspace_bytes(int64_t n);

/* Writes the ascending indices of labels[i] != ignore_index to row_idx_out
 * (capacity n) and their count to count_out[0] (device int64). */
int tlce_compact_rows(const int64_t* labels, int64_t n, int64_t ignore_index,
                      int64_t* row_idx_out, int64_t* count_out,
                      void* workspace, int64_t workspace_bytes, void* stream);

/* The same scan over a boolean mask: the ascending indices of mask[i] != 0
 * (one byte per position, e.g. a torch.bool tensor) and their count.  Device
 * counterpart of `torch.nonzero(supervised_mask.reshape(-1)).flatten()` at the
 * DFlash loss call sites (dllm_parallel/core/models/backbones/dflash/model.py:870-871,
 * dflash2.py:577-578).  Workspace: tlce_compact_workspace_bytes(n). */
int tlce_compact_mask(const uint8_t* mask, int64_t n, int64_t* row_idx_out,
                      int64_t* count_out, void* workspace, int64_t workspace_bytes,
                      void* stream);

/* dst[r, :] = src[row_idx[r], :] for r < m; rows are `row_bytes` long and
 * contiguous in both buffers (index_select along dim 0). */
int tlce_gather_rows(const void* src, const int64_t* row_idx, int64_t m,
                     int64_t row_bytes, void* dst, void* stream);

/* dst[row_idx[r], :] = src[r, :] for r < m.  dst is NOT cleared here; rows not
 * named by row_idx keep their contents (the backward of index_select into a
 * zero-filled buffer, valid because row_idx has no duplicates). */
int tlce_scatter_rows(const void* src, const int64_t* row_idx, int64_t m,
                      int64_t row_bytes, void* dst, void* stream);

/* The compaction gather of the masked-token loss in one launch and without a
 * host read-back of the row count (the reference reads it at
 * `row_indices.numel()`, nemotron/model.py:4247): for r < *row_count
 *   hidden_dst[r] = hidden_src[row_idx[r]], labels_dst[r] = labels_src[row_idx[r]],
 *   weights_dst[r] = weights_src[row_idx[r]]   (weights optional: both NULL or neither);
 * the rows from *row_count up to the next multiple of 64 (at most padded_rows)
 * become zero rows with label ignore_index and weight 0.  row_idx and
 * row_count are what tlce_compact_rows wrote; `capacity` is the number of entries
 * row_idx holds (the most rows there can be; a *row_count outside [0, capacity]
 * is clamped to it), hidden_dst holds padded_rows >= capacity rows of row_bytes
 * bytes, labels_dst / weights_dst padded_rows entries.  Rows past that stay
 * untouched: consumers given row_count never read them. */
int tlce_gather_loss_rows(const void* hidden_src, const int64_t* labels_src,
                          const float* weights_src, const int64_t* row_idx,
                          const int64_t* row_count, int64_t capacity,
                          int64_t padded_rows, int64_t row_bytes,
                          int64_t ignore_index, void* hidden_dst,
                          int64_t* labels_dst, float* weights_dst, void* stream);

/* Zero-fills `bytes` bytes at dst with a kernel (safe inside graph capture). */
int tlce_fill_zero(void* dst, int64_t bytes, void* stream);

/* ---- forward -------------------------------------------------------------
 * Replaces chunked_linear_ce_forward (fused_linear_ce.cpp:94-123).
 *   hidden [m,h], weight [v,h] (vocab-first), labels [m] int64.
 * Outputs: losses (float32; written at row_idx[r] when row_idx != NULL, in
 * which case all n_out entries are first cleared; 0 for ignored rows),
 * lse [m] float32, valid_count [1] float32 (number of rows whose label is not
 * ignore_index).  No [rows, vocab] logits buffer is used: the workspace holds
 * only per-row softmax partials. */
int64_t tlce_forward_workspace_bytes(int64_t m, int64_t h, int64_t v, int dtype);

int tlce_forward(const void* hidden, const void* weight, const float* bias,
                 const int64_t* labels, const int64_t* row_idx,
                 int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                 int64_t ignore_index, int64_t exclude_index,
                 float logit_softcap,
                 float* losses, float* lse, float* valid_count,
                 void* workspace, int64_t workspace_bytes, void* stream);

/* tlce_forward for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same arguments and results as tlce_forward
 * minus the workspace: the per-split softmax partials, the forward's only
 * scratch memory, live in a device array of TLCE_FORWARD_NOALLOC_SCRATCH_BYTES
 * that is part of the library image (every GPU the library runs on holds its
 * copy until the process ends).  The call allocates and frees nothing.
 *   - m beyond TLCE_FORWARD_NOALLOC_MAX_ROWS (more partials than the array
 *     holds) is rejected with an error; nothing is launched then.
 *   - All calls on one GPU share that GPU's array: calls that overlap on one
 *     GPU (two streams, two threads) race.  Nothing in it has to start at zero,
 *     every partial a call reads was written by that call.
 *   - The first call on a device looks the array's address up
 *     (hipGetSymbolAddress) and, like every entry point, raises its kernels'
 *     LDS limit: make one call per device before capturing a graph. */
#define TLCE_FORWARD_NOALLOC_SCRATCH_BYTES (4 << 20)
#define TLCE_FORWARD_NOALLOC_MAX_ROWS 524288

int tlce_forward_noalloc(const void* hidden, const void* weight, const float* bias,
                         const int64_t* labels, const int64_t* row_idx,
                         int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                         int64_t ignore_index, int64_t exclude_index,
                         float logit_softcap,
                         float* losses, float* lse, float* valid_count,
                         void* stream);

/* ---- backward ------------------------------------------------------------
 * Replaces chunked_linear_ce_backward and ..._backward_frozen_weight
 * (fused_linear_ce.cpp:125-207).  grad_weight == NULL selects the
 * frozen-weight variant.
 *   grad_output: float32, [n_out] for TLCE_REDUCTION_NONE, [1] otherwise.
 *   grad_hidden [n_out,h] (dtype): rows named by row_idx receive the gradient
 *   and every other row is cleared; grad_weight [v,h] (dtype);
 *   grad_bias [v] (float32, only when bias != NULL).
 * The gradient of the logits is rounded to `dtype` before the two gradient
 * contractions, as the reference does (fused_linear_ce_cuda.cu:1110-1123).
 * `panel_bytes` bounds the staging panel of vocabulary columns that carries
 * those rounded logit gradients between the kernels (<= 0: default). */
int64_t tlce_backward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                      int dtype, int compute_weight_grad,
                                      int has_bias, int64_t panel_bytes);

int tlce_backward(const void* hidden, const void* weight, const float* bias,
                  const int64_t* labels, const int64_t* row_idx,
                  const float* lse, const float* valid_count,
                  const float* grad_output,
                  int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                  int reduction_code, int64_t ignore_index,
                  int64_t exclude_index, float logit_softcap,
                  void* grad_hidden, void* grad_weight, float* grad_bias,
                  int64_t panel_bytes,
                  void* workspace, int64_t workspace_bytes, void* stream);

/* ---- head stored [h, v] ("dim first") -------------------------------------
 * The reference's extension takes `weight_dim_first` (fused_linear_ce.cpp:104,121)
 * and hands the layout to its GEMMs as a transpose flag.  Here the same: with
 * the entry points below `weight` and `grad_weight` are [h, v] row-major and
 * are read and written in place (the head as a K-major MFMA operand of the two
 * logits contractions, its columns as K-contiguous rows of the grad_hidden
 * contraction, grad_weight produced with the operand roles swapped); no
 * transposed copy of either matrix is made.  Everything else is as for
 * tlce_forward / tlce_backward, same workspaces.
 * Supported where tlce_dim_first_supported(h, v, dtype) returns 1: 16-bit
 * inputs with h and v multiples of 64.  Other shapes are refused with an
 * error; their callers re-lay the head to [v, h] once and use tlce_forward /
 * tlce_backward. */
int tlce_dim_first_supported(int64_t h, int64_t v, int dtype);

int tlce_forward_dim_first(const void* hidden, const void* weight, const float* bias,
                           const int64_t* labels, const int64_t* row_idx,
                           int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                           int64_t ignore_index, int64_t exclude_index,
                           float logit_softcap,
                           float* losses, float* lse, float* valid_count,
                           void* workspace, int64_t workspace_bytes, void* stream);

int tlce_backward_dim_first(const void* hidden, const void* weight, const float* bias,
                            const int64_t* labels, const int64_t* row_idx,
                            const float* lse, const float* valid_count,
                            const float* grad_output,
                            int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                            int reduction_code, int64_t ignore_index,
                            int64_t exclude_index, float logit_softcap,
                            void* grad_hidden, void* grad_weight, float* grad_bias,
                            int64_t panel_bytes,
                            void* workspace, int64_t workspace_bytes, void* stream);

/* ---- masked-token loss ---------------------------------------------------
 * The arithmetic the reference's loss method wraps around the operator
 * (distributed_block_diffusion_loss, nemotron/model.py:2084-2151;
 * _native_token_cross_entropy, :1866-1902), folded into the kernels:
 *   z      = cap(logit_multiplier * hidden . weight^T + bias)
 *            (the reference multiplies a copy of the hidden states, :2084-2086)
 *   loss_r = lse(z_r) - z_r[label_r]                 (0 for ignored rows)
 *   weighted_sum[0] = sum_r token_weights[r] * loss_r      (:2109, :2126-2128)
 * and in the backward, with g = the scale tlce_backward derives from
 * grad_output and reduction_code (for the weighted sum: TLCE_REDUCTION_SUM and
 * grad_output[0] = d objective / d weighted_sum, which carries the caller's
 * `/ valid_token_count * loss_scale`, :2146-2151):
 *   d z_r = (softmax(z_r) - onehot) * g * token_weights[r] * cap'
 *   grad_hidden = logit_multiplier * d z . weight,  grad_weight = logit_multiplier * d z^T . hidden,
 *   grad_bias = sum_r d z_r.
 * No scaled copy of the hidden states, no per-token weighting pass, and the sum
 * is formed in a fixed order (reproducible).
 *   token_weights: float32 [m] aligned with the (compacted) rows, NULL = all 1.
 *   row_count: device int64 or NULL.  With it, m is only the capacity the
 *   launches are sized for: rows r >= *row_count carry no loss and no gradient,
 *   tiles beyond them exit at once, and the kernels re-derive the tile plan
 *   from the real count, so no host synchronisation is needed between the
 *   compaction and the loss.  hidden must then hold round_up(m, 64) rows and
 *   the rows in [*row_count, round_up(*row_count, 64)) must be finite
 *   (tlce_gather_loss_rows writes zeros there).
 *   losses and weighted_sum are each optional (NULL to skip; one of them must
 *   be given): per-token losses at row_idx positions as tlce_forward writes
 *   them, and the weighted sum.  logit_multiplier must be positive.
 *   Workspaces: tlce_masked_loss_forward_workspace_bytes for the forward,
 *   tlce_backward_workspace_bytes for the backward. */
int64_t tlce_masked_loss_forward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                                 int dtype, int dynamic_rows);

int tlce_masked_loss_forward(const void* hidden, const void* weight, const float* bias,
                             const int64_t* labels, const float* token_weights,
                             const int64_t* row_idx, const int64_t* row_count,
                             int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                             int64_t ignore_index, int64_t exclude_index,
                             float logit_softcap, float logit_multiplier,
                             float* losses, float* lse, float* valid_count,
                             float* weighted_sum,
                             void* workspace, int64_t workspace_bytes, void* stream);

int tlce_masked_loss_backward(const void* hidden, const void* weight, const float* bias,
                              const int64_t* labels, const float* token_weights,
                              const int64_t* row_idx, const int64_t* row_count,
                              const float* lse, const float* valid_count,
                              const float* grad_output,
                              int64_t m, int64_t n_out, int64_t h, int64_t v, int dtype,
                              int reduction_code,
                              int64_t ignore_index, int64_t exclude_index,
                              float logit_softcap, float logit_multiplier,
                              void* grad_hidden, void* grad_weight, float* grad_bias,
                              int64_t panel_bytes,
                              void* workspace, int64_t workspace_bytes, void* stream);

/* ---- vocabulary shards ---------------------------------------------------
 * Replace vocab_parallel_ce_forward_local / vocab_parallel_ce_backward_local
 * (fused_linear_ce.cpp:209-265; fused_vocab_parallel_ce_forward_cuda and
 * vocab_parallel_ce_stats_kernel, fused_linear_ce_cuda.cu:292-365,1174-1268):
 * the tensor-parallel form of the loss, where a rank owns the weight rows
 * [vocab_start, vocab_start + v_local) and labels / exclude_index stay global
 * ids.  The caller combines the per-row statistics of all shards (one MAX and
 * one SUM reduction) into the global lse and hands it to the backward.
 *   forward_local: local_max[m] = max over the shard's non-excluded columns
 *   (-inf if none), local_sum[m] = sum exp(z - local_max), target_logits[m] =
 *   logit of the label if this shard owns it and the row is not ignored, else
 *   0 (-inf if the label is the excluded column and local), valid_count[1].
 *   Every row gets statistics, ignored ones too, as in the reference.
 *   backward_local: as tlce_backward with lse = global_lse; grad_hidden [m,h]
 *   is this shard's partial sum (the caller sums over shards), grad_weight
 *   [v_local,h] and grad_bias [v_local] are complete.
 * Workspaces: tlce_forward_workspace_bytes / tlce_backward_workspace_bytes
 * with v = v_local. */
int tlce_forward_local(const void* hidden, const void* weight, const float* bias,
                       const int64_t* labels, int64_t m, int64_t h,
                       int64_t v_local, int dtype, int64_t vocab_start,
                       int64_t ignore_index, int64_t exclude_index,
                       float logit_softcap, float* local_max, float* local_sum,
                       float* target_logits, float* valid_count,
                       void* workspace, int64_t workspace_bytes, void* stream);

int tlce_backward_local(const void* hidden, const void* weight, const float* bias,
                        const int64_t* labels, const float* global_lse,
                        const float* valid_count, const float* grad_output,
                        int64_t m, int64_t h, int64_t v_local, int dtype,
                        int reduction_code, int64_t vocab_start,
                        int64_t ignore_index, int64_t exclude_index,
                        float logit_softcap, void* grad_hidden, void* grad_weight,
                        float* grad_bias, int64_t panel_bytes, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* ---- streaming soft embedding ---------------------------------------------
 * Replaces streaming_soft_embedding(_from_shards)
 * (dllm_parallel/core/kernels/streaming_soft_embedding.py:60-148):
 *   out[r] = embedding_scale * softmax(cap(hidden[r] . weight^T)) . weight
 * forward-only, without a logits buffer: the forward tile loop yields lse, the
 * probability panels (rounded to `dtype`, as the reference rounds them before
 * its second matmul) are contracted with the weight rows in float32: three
 * contractions.  Under a soft cap of at most 40 (bf16, h and v multiples of 64)
 * two suffice: capped logits lie in [-cap, cap], so exp(logit - cap) needs no
 * row maximum; it is written for a block of rows over the whole vocabulary
 * into a panel of panel_bytes (0: 2.5 GiB), contracted with the weight rows, and
 * the result divided by the row's sum.  Without such a cap the same operands
 * take two contractions as well: one pass writes exp2(logit2 - the exact maximum
 * of the token's 256-entry vocabulary tile) with the tile's softmax partials,
 * the entries are normalised per (token, tile) once the lse is merged, then
 * contracted.  The workspace query covers every sequence.
 *   hidden [m,h], weight [v,h], out [m,h], all `dtype`. */
int64_t tlce_soft_embedding_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                            int dtype, int64_t panel_bytes);

int tlce_soft_embedding(const void* hidden, const void* weight, int64_t m,
                        int64_t h, int64_t v, int dtype, float logit_softcap,
                        float embedding_scale, void* out, int64_t panel_bytes,
                        void* workspace, int64_t workspace_bytes, void* stream);

/* ---- frozen-head forward KL -------------------------------------------------
 * Replaces dflash_frozen_kl_forward / dflash_frozen_kl_backward
 * (fused_linear_ce.cpp:267-304; fused_linear_ce_cuda.cu:367-480,1270-1509):
 *   losses[r] = sum_v p_t (log p_t - log p_d),  p_x = softmax(cap(hidden_x[r] . weight_x^T))
 * for a draft and a teacher head over one vocabulary; only the draft hidden
 * states get a gradient,
 *   grad_hidden = ((p_d - p_t) * grad_output[r] * cap'(z_d)) . draft_weight,
 * with the logit gradient rounded to `dtype` before the contraction, like the
 * reference.  No logits buffer: the teacher probabilities cross memory in the
 * same bounded vocabulary panels as the cross-entropy backward (rounded to
 * `dtype`; the loss is accumulated as the generalised KL sum t log(t/q) - t + q,
 * which is insensitive to that rounding to first order).  Forward: one
 * statistics pass over the teacher head, then per panel the teacher
 * probabilities and one pass over the draft head that yields both the loss
 * terms and the draft's softmax statistics.
 * teacher_probabilities (optional, both calls): a caller-owned buffer of
 * tlce_kl_teacher_probabilities_bytes (2 bytes per padded row and vocabulary
 * entry: 2.5 GB at m = 8192, v = 151936) that the forward fills with the teacher
 * probabilities of every panel and the backward reads instead of producing them
 * again: 5 contractions per forward + backward instead of 6 (the reference runs
 * 5 GEMMs, fused_linear_ce_cuda.cu:1270-1509).  NULL: nothing is kept.
 *   draft_hidden [m,h_draft], draft_weight [v,h_draft], teacher_hidden
 *   [m,h_teacher], teacher_weight [v,h_teacher], all `dtype`; losses,
 *   draft_lse, teacher_lse, grad_output: float32 [m]; grad_hidden [m,h_draft]. */
int64_t tlce_kl_workspace_bytes(int64_t m, int64_t h_draft, int64_t h_teacher,
                                int64_t v, int dtype, int64_t panel_bytes);

int tlce_kl_forward(const void* draft_hidden, const void* draft_weight,
                    const void* teacher_hidden, const void* teacher_weight,
                    int64_t m, int64_t h_draft, int64_t h_teacher, int64_t v,
                    int dtype, float logit_softcap, float* losses,
                    float* draft_lse, float* teacher_lse,
                    void* teacher_probabilities, int64_t panel_bytes,
                    void* workspace, int64_t workspace_bytes, void* stream);

int64_t tlce_kl_teacher_probabilities_bytes(int64_t m, int64_t h_draft,
                                            int64_t h_teacher, int64_t v, int dtype);

/* The forward with the gradient formed in it: 3 contractions per forward +
 * backward.  A pass over a head holds every logit of a tile in registers; it
 * writes exp2(logit2 - the exact maximum of the token's 256-entry vocabulary
 * tile) <= 1 in bf16 into a panel over the whole vocabulary and leaves the
 * tile's (maximum, sum), so that softmax = entry * exp2(tile maximum - lse2)
 * per (token, tile) once the lse is merged.  One such pass over the teacher
 * head replaces its statistics pass and its probabilities pass; the draft pass
 * reads the teacher's entries, accumulates the loss terms and writes its own
 * entries into a second panel; one elementwise pass then forms
 *   g[r, v] = entry_d * exp2(max_d - lse2_d[r]) - entry_t * exp2(max_t - lse2_t[r])
 * (times cap'(z) under a soft cap, z re-derived from the entry), and one
 * contraction with the draft head leaves
 *   unit_grad_hidden_f32[r, :] = d losses[r] / d draft_hidden[r, :]   float32 [m, h_draft].
 * The backward is tlce_apply_grad_output(unit, NULL, NULL, NULL, grad_output, NULL,
 * m, m, h_draft, v, dtype, TLCE_REDUCTION_NONE, grad_hidden, NULL, stream).
 * bf16, a soft cap between 10 and 40 or none, both hidden sizes and v multiples of 64
 * (tlce_kl_gradient_in_forward_supported); rows are taken in blocks of the 2.5 GiB
 * panel budget one after the other, and the workspace holds both panels of a block
 * (2 x 2 bytes per padded row and vocabulary entry). */
int tlce_kl_gradient_in_forward_supported(int64_t m, int64_t h_draft,
                                          int64_t h_teacher, int64_t v, int dtype,
                                          float logit_softcap);

int64_t tlce_kl_forward_with_gradient_workspace_bytes(int64_t m, int64_t h_draft,
                                                      int64_t h_teacher, int64_t v,
                                                      int dtype, int64_t panel_bytes);

int tlce_kl_forward_with_gradient(
    const void* draft_hidden, const void* draft_weight, const void* teacher_hidden,
    const void* teacher_weight, int64_t m, int64_t h_draft, int64_t h_teacher,
    int64_t v, int dtype, float logit_softcap, float* losses, float* draft_lse,
    float* teacher_lse, float* unit_grad_hidden_f32, int64_t panel_bytes,
    void* workspace, int64_t workspace_bytes, void* stream);

int tlce_kl_backward(const void* draft_hidden, const void* draft_weight,
                     const void* teacher_hidden, const void* teacher_weight,
                     const float* draft_lse, const float* teacher_lse,
                     const float* grad_output, const void* teacher_probabilities,
                     int64_t m, int64_t h_draft,
                     int64_t h_teacher, int64_t v, int dtype, float logit_softcap,
                     void* grad_hidden, int64_t panel_bytes, void* workspace,
                     int64_t workspace_bytes, void* stream);

/* ---- frozen-head cross entropy with exact top-k ---------------------------
 * Replaces dflash_ce_topk_forward / dflash_ce_topk_backward
 * (fused_linear_ce.cpp:306-354; fused_linear_ce_cuda.cu:482-599,1511-1773;
 * torch form in dllm_parallel/core/kernels/dflash_linear_topk.py:100-225):
 *   z = cap(output_multiplier * hidden . weight^T),  losses = lse(z) - z[label],
 *   probabilities = exp(-losses), top_values / top_ids = the top_k largest z of
 *   every row, sorted descending (ties towards the smaller id), lse [m].
 * The logits cross memory once, in float32, in vocabulary panels bounded by
 * `panel_bytes`; a per-row scan folds each panel into the running softmax
 * statistics and the running top-k list.  top_k <= 256.
 * Backward (hidden only; the head is frozen):
 *   grad_hidden = (softmax(z) * ce_scale[r] * dz/draw) . weight
 *                 - ce_scale[r] * dz/draw[label] * weight[label]
 *                 + sum_j grad_top_values[r,j] * dz/draw[id_j] * weight[id_j]
 * with ce_scale = grad_loss - grad_probability * probability (the caller forms
 * it) and grad_top_values optional (NULL: no such term).
 *   hidden [m,h], weight [v,h] (`dtype`), labels [m] int64 in [0, v);
 *   float32: losses, probabilities, lse, ce_scale [m], top_values and
 *   grad_top_values [m,top_k]; top_ids int64 [m,top_k]; grad_hidden [m,h]. */
int64_t tlce_ce_topk_forward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                             int dtype, int64_t panel_bytes);
int64_t tlce_ce_topk_backward_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                              int dtype, int64_t panel_bytes);

int tlce_ce_topk_forward(const void* hidden, const void* weight,
                         const int64_t* labels, int64_t m, int64_t h, int64_t v,
                         int dtype, int top_k, float output_multiplier,
                         float logit_softcap, float* losses, float* probabilities,
                         float* top_values, int64_t* top_ids, float* lse,
                         int64_t panel_bytes, void* workspace,
                         int64_t workspace_bytes, void* stream);

int tlce_ce_topk_backward(const void* hidden, const void* weight,
                          const int64_t* labels, const float* lse,
                          const int64_t* top_ids, const float* ce_scale,
                          const float* grad_top_values, int64_t m, int64_t h,
                          int64_t v, int dtype, int top_k, float output_multiplier,
                          float logit_softcap, void* grad_hidden,
                          int64_t panel_bytes, void* workspace,
                          int64_t workspace_bytes, void* stream);

/* The same pair with the softmax part of the gradient formed in the forward
 * (dflash_ce_topk_forward + dflash_ce_topk_backward, fused_linear_ce.cpp:306-354,
 * whose backward recomputes the logits): while a float32 logits panel exists,
 * exp(z - the row's largest logit so far) * dz/draw is written in bf16 into a
 * panel over the whole vocabulary (2 bytes per row and vocabulary entry inside
 * the workspace; panels written before a row's maximum grew are rescaled
 * afterwards), and one contraction with the weight rows leaves
 *   unit_grad_hidden_f32[r, :] = d lse[r] / d hidden[r, :]      float32 [m, h].
 * tlce_ce_topk_apply_gradient then forms, in one pass over rows,
 *   grad_hidden[r, :] = ce_scale[r] * unit[r, :]
 *                       - ce_scale[r] * dz/draw[label] * weight[label]
 *                       + sum_j grad_top_values[r,j] * dz/draw[id_j] * weight[id_j]
 * rounded once: 2 contractions per step instead of 3.  bf16, h and v multiples
 * of 64 (tlce_ce_topk_gradient_in_forward_supported); rows are taken in blocks
 * of the 2.5 GiB panel budget (8192 rows at v = 151936), one after the other on
 * one workspace; panel_bytes bounds the float32 logits panels as in
 * tlce_ce_topk_forward. */
int tlce_ce_topk_gradient_in_forward_supported(int64_t m, int64_t h, int64_t v,
                                               int dtype);

int64_t tlce_ce_topk_forward_with_gradient_workspace_bytes(int64_t m, int64_t h,
                                                           int64_t v, int dtype,
                                                           int64_t panel_bytes);

int tlce_ce_topk_forward_with_gradient(
    const void* hidden, const void* weight, const int64_t* labels, int64_t m,
    int64_t h, int64_t v, int dtype, int top_k, float output_multiplier,
    float logit_softcap, float* losses, float* probabilities, float* top_values,
    int64_t* top_ids, float* lse, float* unit_grad_hidden_f32,
    int64_t panel_bytes, void* workspace, int64_t workspace_bytes, void* stream);

int tlce_ce_topk_apply_gradient(const float* unit_grad_hidden_f32,
                                const void* hidden, const void* weight,
                                const int64_t* labels, const int64_t* top_ids,
                                const float* ce_scale, const float* grad_top_values,
                                int64_t m, int64_t h, int64_t v, int dtype,
                                int top_k, float output_multiplier,
                                float logit_softcap, void* grad_hidden,
                                void* stream);

/* ---- per-sample loss numerators of the DFlash loss method -----------------
 * Replaces `numerators.scatter_add_(0, sample_indices, token_loss * position_weights)`
 * with sample_indices = valid_indices // tokens_per_sample
 * (dllm_parallel/core/models/backbones/dflash/model.py:918-937):
 *   out[s] = sum of values[r] * weights[r] over the compacted rows r whose
 *            position row_idx[r] lies in [s * segment_length, (s + 1) * segment_length)
 * for s < n_segments, float32.  row_idx (int64, ascending, m entries: what
 * tlce_compact_mask / tlce_compact_rows wrote) makes each sample's rows one
 * contiguous run, which one workgroup adds in a fixed order: no atomics, the
 * same bits on every run.  weights == NULL: plain sums.  row_count (device
 * int64, optional): the real number of rows when m is only a capacity. */
int tlce_segment_weighted_sum(const float* values, const float* weights,
                              const int64_t* row_idx, const int64_t* row_count,
                              int64_t m, int64_t segment_length, int64_t n_segments,
                              float* out, void* stream);

/* ---- forward that also leaves the gradients: 3 contractions, not 4 ---------
 * Replaces the pair fused_linear_ce_forward + fused_linear_ce_backward
 * (dllm_parallel/csrc/fused_linear_ce.cpp:94-207) for callers whose upstream
 * gradient is one number (reduction "sum" / "mean", or a weighted sum of the
 * token losses): the reference's backward recomputes the logits of every block
 * (fused_linear_ce_cuda.cu:618-791), the plain entry points here do the same
 * by vocabulary panels.  This entry point forms the gradients of
 *     S = sum_r token_weights[r] * loss[r]
 * while the logits of a block of rows exist:
 *     grad_hidden_f32[r, :]  = dS / d hidden[r, :]      [m, h] float32, compact rows
 *     grad_weight_f32[v, :]  = dS / d weight[v, :]      [v, h] float32 (NULL: frozen head)
 * and writes losses / lse / valid_count as tlce_forward does (losses unweighted;
 * lse is 0, not computed, for rows whose label is ignore_index).
 * tlce_apply_grad_output then multiplies both by the upstream gradient
 * (grad_output[0], divided by valid_count[0] for TLCE_REDUCTION_MEAN), rounds
 * them once to the input dtype, and un-compacts grad_hidden through row_idx
 * into [n_out, h] (other rows zero).  With TLCE_REDUCTION_NONE the upstream
 * gradient is one float per output row, grad_output[n_out] (row r of the compact
 * rows reads grad_output[row_idx[r]]): call the forward without token_weights;
 * grad_hidden rows are scaled one by one, and grad_weight, which needs the
 * upstream gradient inside its contraction, is only available through
 * tlce_grad_weight_from_panel, i.e. when all rows form one block
 * (grad_weight_f32 must be NULL here).  No bias, head stored [v, h], bf16 inputs
 * with h and v multiples of 64 (tlce_fused_gradients_supported); everything else
 * goes through tlce_forward / tlce_backward (f16 included: its exponent range
 * cannot hold exp(logit - reference) and the row sums of it).
 *
 * Rows are taken in blocks of as many rows as a panel of panel_bytes (0: 2.5 GiB)
 * holds over the whole vocabulary (tlce_query_fused_plan); the panel holds
 * exp(logit - reference) in bf16, the reference being the label's
 * logit of the row.  A block in which some row's largest logit lies more than
 * 40 above its reference is produced a second time with the exact
 * row maxima as references; the decision is taken on the device, the second
 * try's launches are always made and do nothing otherwise.
 * logit_multiplier > 0 scales the raw dot products (1: plain operator).
 * row_count (device int64, optional, needs row_idx): the real number of rows
 * when m is only the capacity the launches and buffers are sized for; as in
 * tlce_masked_loss_*, workgroups past the count exit at once and nothing needs
 * the host, so compaction, this call and tlce_apply_grad_output record into one
 * HIP graph that serves any mask. */
int tlce_fused_gradients_supported(int64_t h, int64_t v, int dtype);

int tlce_query_fused_plan(int64_t m, int64_t h, int64_t v, int dtype,
                          int64_t panel_bytes, int64_t* block_rows, int* n_blocks,
                          int* grad_hidden_k_splits);

int64_t tlce_forward_with_gradients_workspace_bytes(int64_t m, int64_t h, int64_t v,
                                                    int dtype, int compute_weight_grad,
                                                    int64_t panel_bytes);

int tlce_forward_with_gradients(const void* hidden, const void* weight,
                                const int64_t* labels, const int64_t* row_idx,
                                const float* token_weights, const int64_t* row_count,
                                int64_t m, int64_t n_out,
                                int64_t h, int64_t v, int dtype, int64_t ignore_index,
                                int64_t exclude_index, float logit_softcap,
                                float logit_multiplier, float* losses, float* lse,
                                float* valid_count, float* grad_hidden_f32,
                                float* grad_weight_f32, int64_t panel_bytes,
                                void* workspace, int64_t workspace_bytes, void* stream);

int tlce_apply_grad_output(const float* grad_hidden_f32, const float* grad_weight_f32,
                           const int64_t* row_idx, const int64_t* row_count,
                           const float* grad_output,
                           const float* valid_count, int64_t m, int64_t n_out,
                           int64_t h, int64_t v, int dtype, int reduction_code,
                           void* grad_hidden, void* grad_weight, void* stream);

/* One block of rows only (tlce_query_fused_plan: n_blocks == 1): the grad_weight
 * contraction of tlce_forward_with_gradients postponed until the upstream
 * gradient is known.  Call the forward with grad_weight_f32 = NULL (as for a
 * frozen head) on a workspace sized with compute_weight_grad = 1 and keep that
 * workspace untouched; the panel in it still holds exp(logit - reference) of
 * every row, so
 *     grad_weight[v, :] = sum_r panel[r, v] * (g * s_r * hidden[r, :])
 * (g = grad_output[0], over valid_count[0] for the mean; grad_output[row_idx[r]],
 * or grad_output[r] without row_idx, for TLCE_REDUCTION_NONE; s_r the row factor
 * the forward left in the workspace) is stored directly in the input dtype: no
 * float32 [v, h] accumulator and no pass that scales and rounds it.  m, h, v,
 * dtype, panel_bytes, row_idx and row_count as given to the forward.  May be called
 * again on the same workspace (it rewrites only its own operand area). */
int tlce_grad_weight_from_panel(const void* hidden, const int64_t* row_idx,
                                const int64_t* row_count, const float* grad_output, const float* valid_count,
                                int64_t m, int64_t h, int64_t v, int dtype,
                                int reduction_code, void* grad_weight,
                                int64_t panel_bytes, void* forward_workspace,
                                int64_t workspace_bytes, void* stream);

/* ---- introspection used by the benchmark and the tests -------------------
 * Tile plan the host scheduler would use for a problem; any pointer may be
 * NULL.  `engine` is 2 for the bf16/f16 MFMA kernels with direct-to-LDS loads
 * (h a multiple of 32), 1 for the register-staged MFMA kernels (h a multiple of
 * 8), 0 for the generic float32-FMA kernels (float32 inputs, other h). */
int tlce_query_plan(int64_t m, int64_t h, int64_t v, int dtype,
                    int compute_weight_grad, int64_t panel_bytes,
                    int* engine, int64_t* tile, int64_t* forward_vocab_splits,
                    int64_t* panel_columns, int64_t* n_panels,
                    int64_t* grad_hidden_k_splits);

/* ---- per-kernel timing (benchmark support; no reference counterpart) -----
 * Between tlce_profile_begin() and tlce_profile_end() every kernel the calling
 * thread launches through this library is bracketed by HIP events on its
 * stream.  tlce_profile_end waits for them and adds up, per kernel class,
 * the elapsed milliseconds and the launch count.  Classes:
 *   0 forward logits+softmax-stats tiles   1 per-row loss merge
 *   2 backward logit-gradient panel tiles  3 grad_hidden contraction
 *   4 grad_weight contraction              5 operand transposes
 *   6 fills, scales and casts             7 exponentiated-logits panel tiles
 * The events allocate driver resources: not for use under graph capture. */
#define TLCE_PROFILE_CLASSES 8
int tlce_profile_begin(void);
int tlce_profile_end(double* class_ms, int64_t* class_launches, int n_classes);

#ifdef __cplusplus
}
#endif

#endif /* TLCE_H_ */

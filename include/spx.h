/*
 * C-ABI of libspx_hip.so -- the MI355X (gfx950) kernels behind the draft-model
 * training hot path of vllm-project/speculators.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its comment says "host";
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     every entry point only enqueues work on that stream and returns;
 *   - the caller owns every buffer, workspaces included; entry points allocate
 *     nothing;
 *   - the return value is 0 on success, 1 for a rejected argument, 2 for a HIP
 *     launch error; spx_last_error() holds the message (thread-local);
 *   - `dtype` codes: 0 = bf16, 1 = f32.  Mask element codes (`*_kind`):
 *     0 = 1-byte (bool / uint8), 1 = int32, 2 = int64, 3 = f32, 4 = bf16.
 *   - reference citations are relative to src/speculators/ of the reference.
 */
#ifndef SPX_H
#define SPX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPX_DTYPE_BF16 0
#define SPX_DTYPE_F32 1

#define SPX_KIND_U8 0
#define SPX_KIND_I32 1
#define SPX_KIND_I64 2
#define SPX_KIND_F32 3
#define SPX_KIND_BF16 4

/* loss selector; the same five reductions as the `OP` constexpr of
 * losses/fused.py:38-46 */
#define SPX_LOSS_KL 0
#define SPX_LOSS_RKL 1
#define SPX_LOSS_JSD 2
#define SPX_LOSS_CE 3
#define SPX_LOSS_TV 4

int spx_version(void);
const char* spx_last_error(void); /* host string, valid until the next failing call on this thread */

/* ---------------------------------------------------------------- vocabulary
 * out[r, i] = full[r, i + d2t[i]]  (bit-exact copy of bf16 / f32 elements).
 * Replaces the t2d row-slice of the verifier head, model.py:161-169, with a
 * gather of full-vocabulary verifier logits through the d2t offset table of
 * train/vocab_mapping.py:86-96.  Indices outside [0, vt) are rejected on the
 * device by writing -inf (they cannot occur for a table built by the
 * reference). */
int spx_vocab_gather(const void* full, int64_t ld_full, const int64_t* d2t,
                     void* out, int64_t ld_out, int64_t rows, int64_t vd,
                     int64_t vt, int dtype, void* stream);

/* ---------------------------------------------------------------- fused loss
 * One streaming pass per row over a draft row and a target row:
 *   loss[r]       row loss selected by `op` (fp32)
 *   lse_draft[r]  log-sum-exp of the draft row,  lse_target[r] of the target row
 *   extra[r]      kl/rkl: the row loss; jsd: KL(q||m); tv: sum of q where q<=p;
 *                 ce: unused (the label is argmax_target[r])
 *   argmax_draft[r], argmax_target[r]  first-index argmax (torch.argmax rule)
 * Replaces loss_forward_kernel (losses/fused.py:91-175) and the two
 * torch.argmax calls of compute_metrics (models/eagle3/metrics.py:100-101,
 * models/dflash/metrics.py:77-78).  Row r of `logits` is paired with row r of
 * `targets`; the TTT shift of align_for_step (models/eagle3/metrics.py:16-48)
 * is a pointer offset made by the caller.  ld_* are row strides in elements.
 * The argmax outputs may be NULL.
 * reuse_target_stats != 0 (kl and ce only; ignored for the others): lse_target
 * and argmax_target are INPUTS holding the statistics of the same target rows
 * from an earlier call -- the verifier row is the same at every TTT step, only
 * shifted -- so the target max / sum / arg-max are not recomputed, and ce does
 * not read the target rows at all: `targets` may then be NULL (the arg-max can come
 * from spx_gemm_bf16_nt_stats, and the verifier's logits never exist in memory). */
int spx_fused_vocab_loss_fwd(int op, const void* logits, int64_t ld_logits,
                             const void* targets, int64_t ld_targets,
                             int64_t rows, int64_t vocab, int dtype,
                             float* loss, float* lse_draft, float* lse_target,
                             float* extra, int32_t* argmax_draft,
                             int32_t* argmax_target, int reuse_target_stats,
                             void* stream);

/* The whole per-row work of one TTT step in ONE streaming pass: spx_fused_vocab_loss_fwd plus
 *   - d2t != NULL: `targets` holds FULL-vocabulary verifier rows (vt columns, row stride
 *     ld_targets) and target element i is read at column i + d2t[i] -- the d2t / t2d mapping
 *     of model.py:161-169 and train/vocab_mapping.py:86-96 applied while streaming, no
 *     [rows, vocab] copy of the targets is needed first.  `gathered` (may be NULL) receives
 *     that draft-vocabulary row (bit-exact copy), for the later TTT steps and the backward,
 *     which then stream vocab-wide rows.  Columns outside [0, vt) read as -inf.
 *     reuse_target_stats must be 0 in this form.
 *   - counts != NULL (int32[3], zeroed by the caller): the row's part of the acceptance chain
 *     of compute_accuracy_single_step (models/metrics.py:6-36) as called from compute_metrics
 *     (models/eagle3/metrics.py:100-117).  With m = mask[r] != 0 (NULL: 1), was =
 *     prev_correct[r] != 0 (NULL: 1), now = was && argmax_draft[r] == argmax_target[r]:
 *       counts[0] += m && now   (full_correct = cond_correct)
 *       counts[1] += m          (full_total)
 *       counts[2] += was        (cond_total, counted before the update)
 *       prev_correct[r] = now   (in place, in prev_correct's own element type)
 *     Integer atomics: the result does not depend on the order in which rows finish.
 *     Needs both arg-max outputs.  spx_ttt_step_mean turns the counts and the row losses
 *     into the step's scalars.
 * Replaces, together, the t2d row slice (model.py:161-169), loss_forward_kernel
 * (losses/fused.py:91-175), both torch.argmax calls and compute_accuracy_single_step. */
int spx_vocab_loss_step_fwd(int op, const void* logits, int64_t ld_logits,
                            const void* targets, int64_t ld_targets, const int64_t* d2t,
                            int64_t vt, void* gathered, int64_t ld_gathered, int64_t rows,
                            int64_t vocab, int dtype, float* loss, float* lse_draft,
                            float* lse_target, float* extra, int32_t* argmax_draft,
                            int32_t* argmax_target, int reuse_target_stats,
                            const void* mask, int mask_kind, void* prev_correct,
                            int prev_kind, int32_t* counts, void* stream);

/* The row pass of a TTT step that also leaves the gradient of the logits behind (kl and ce, bf16,
 * vocab a multiple of 8 and at most 32768, 16-byte aligned rows): a workgroup holds the whole row
 * pair in registers, so logits and targets are read ONCE for loss_forward_kernel and
 * loss_backward_kernel together (losses/fused.py:91-235) -- three row transfers per live row
 * instead of five.  Outputs and the acceptance chain as for spx_vocab_loss_step_fwd (no d2t
 * form); additionally, for every row r with row_map[r] >= 0 (spx_pack_row_map of the loss mask),
 *   grad_logits[row_map[r], :] = softmax(logits[r]) - softmax(targets[r])          (kl)
 *                                softmax(logits[r]) - onehot(argmax targets[r])     (ce)
 * i.e. the gradient for a row weight of ONE: what follows is linear in the rows, so the weight
 * the reduction behind the loss gives row r is applied to the result of the input-gradient
 * product (spx_unpack_rows_scaled).  Rows mapped to -1 get no gradient row; with
 * reuse_target_stats their target row is not read and their loss and lse_draft are written as 0
 * (a masked row's loss enters no sum), their arg-max outputs and chain update are as for any
 * row. */
int spx_vocab_loss_step_fwd_grad(int op, const void* logits, int64_t ld_logits,
                                 const void* targets, int64_t ld_targets, int64_t rows,
                                 int64_t vocab, float* loss, float* lse_draft,
                                 float* lse_target, float* extra, int32_t* argmax_draft,
                                 int32_t* argmax_target, int reuse_target_stats,
                                 const void* mask, int mask_kind, void* prev_correct,
                                 int prev_kind, int32_t* counts, const int32_t* row_map,
                                 void* grad_logits, int64_t ld_grad, void* stream);

/* grad_logits[r, :] = g_r * dL_r/dlogits, g_r = row_grad[r] * (*scale)
 * (scale may be NULL = 1).  Rows with g_r == 0 are written as exact zeros
 * without reading the inputs.  Closed forms of losses/fused.py:11-18; replaces
 * loss_backward_kernel (losses/fused.py:177-235).  grad dtype = `dtype`. */
int spx_fused_vocab_loss_bwd(int op, const void* logits, int64_t ld_logits,
                             const void* targets, int64_t ld_targets,
                             int64_t rows, int64_t vocab, int dtype,
                             const float* lse_draft, const float* lse_target,
                             const float* extra, const int32_t* argmax_target,
                             const float* row_grad, const float* scale,
                             void* grad_logits, int64_t ld_grad, void* stream);

/* The same gradient with the live rows packed to the front: row r goes to row
 * row_map[r] of grad_logits, rows with row_map[r] < 0 (zero gradient: masked out
 * of the loss, losses/utils.py:233-304) are not written.  Feeds
 * spx_gemm_bf16_nt_rows, which skips them in the lm_head input-gradient product.
 * No counterpart in the reference, where that product runs over all rows. */
int spx_fused_vocab_loss_bwd_packed(int op, const void* logits, int64_t ld_logits,
                                    const void* targets, int64_t ld_targets,
                                    int64_t rows, int64_t vocab, int dtype,
                                    const float* lse_draft, const float* lse_target,
                                    const float* extra, const int32_t* argmax_target,
                                    const float* row_grad, const float* scale,
                                    const int32_t* row_map, void* grad_logits,
                                    int64_t ld_grad, void* stream);

/* Cross-entropy of full-vocabulary logits against integer labels, the loss of
 * the multi-token-prediction path: loss[r] = logsumexp(logits[r, :]) -
 * logits[r, labels[r]], 0 where labels[r] == ignore_index (such rows are not
 * read unless argmax is requested); lse[r] is kept for the backward; argmax
 * (may be NULL) = first index of the row maximum.  A label outside [0, vocab)
 * other than ignore_index gives NaN.  fp32 statistics whatever `dtype` is.
 * Replaces F.cross_entropy(logits.permute(0, 2, 1), targets, ignore_index=-100,
 * reduction="none") of models/mtp/core.py:204-216. */
int spx_label_ce_fwd(const void* logits, int64_t ld_logits, const int64_t* labels,
                     int64_t rows, int64_t vocab, int dtype, int64_t ignore_index,
                     float* loss, float* lse, int32_t* argmax, void* stream);

/* The label cross-entropy of rows whose log-sum-exp is known already (spx_gemm_bf16_nt_stats
 * computes it in the head product's epilogue): loss[r] = lse[r] - logits[r, labels[r]], 0 for an
 * ignored label, NaN for a label outside [0, vocab) -- the values spx_label_ce_fwd returns,
 * with one element of every row read instead of the row (models/mtp/core.py:204-216). */
int spx_label_ce_from_lse(const void* logits, int64_t ld_logits, const int64_t* labels,
                          int64_t rows, int64_t vocab, int dtype, int64_t ignore_index,
                          const float* lse, float* loss, void* stream);

/* dlogits[r, j] = grad_rows[r] * (softmax(logits[r, :])[j] - [j == labels[r]]);
 * rows with grad_rows[r] == 0 or an ignored label are exact zeros and are not
 * read.  The autograd backward of the call above (models/mtp/core.py:204-218). */
int spx_label_ce_bwd(const void* logits, int64_t ld_logits, const int64_t* labels,
                     const float* lse, const float* grad_rows, int64_t rows,
                     int64_t vocab, int dtype, int64_t ignore_index, void* dlogits,
                     int64_t ld_out, void* stream);

/* The same gradient with the live rows packed to the front: row r is written to
 * row row_map[r] of dlogits, rows with row_map[r] < 0 are not written at all
 * (their gradient is zero: ignored label or grad_rows[r] == 0; the caller builds
 * the map as a running count of the live rows).  Feeds spx_gemm_bf16_nt_rows, which
 * then skips the dead rows of the lm_head input-gradient product.  No counterpart
 * in the reference, where that product runs over all rows. */
int spx_label_ce_bwd_packed(const void* logits, int64_t ld_logits, const int64_t* labels,
                            const float* lse, const float* grad_rows, int64_t rows,
                            int64_t vocab, int dtype, int64_t ignore_index,
                            const int32_t* row_map, void* dlogits, int64_t ld_out,
                            void* stream);

/* Batch layout producer: packs `n_docs` samples, staged back to back in the layout
 * of the hidden-state files (`src_hs [n_src_rows, layers + 1, hidden]`, bf16 or fp32,
 * with `src_ids [n_src_rows]` int64 and `src_mask [n_src_rows]` of `mask_elem`-byte
 * elements), into the one-row batch the draft models consume.  Output row r of
 * document d (the last d with out_start[d] <= r < out_start[n_docs]), offset
 * o = r - out_start[d]:
 *   out_aux [r, :]  = bf16(src_hs[src_start[d] + o, 0:layers, :])        (may be NULL)
 *   out_last[r, :]  = bf16(src_hs[src_start[d] + o + shift, layers, :])  (may be NULL)
 *   out_ids / out_mask [r] = src_ids / src_mask [src_start[d] + o + shift]
 *   out_pos [r] = src_pos ? src_pos[src_start[d] + o + shift] : o + shift
 *   out_doc [r] = d
 * rows r >= out_start[n_docs] are padding: zeros, out_doc = -1.  `src_start` and
 * `out_start` are device int64 arrays of n_docs + 1 entries (out_start[0] = 0,
 * non-decreasing, out_start[n_docs] <= max_len); a row whose source index falls outside
 * [0, n_src_rows) is written as padding, never read.  shift = 1 gives the EAGLE3
 * alignment (x[i+1], g[i], y[i+1], mask[i+1]), shift = 0 the DFlash / MTP one.
 * Replaces, on the device, CollateFn.__call__ (train/data.py:323-393) composed with
 * shift_batch (models/eagle3/data.py:8-44) or shift_batch_mtp (models/mtp/data.py:6-18)
 * and the layer split of ArrowDataset._get_raw_data (train/data.py:293-303). */
int spx_pack_batch(const void* src_hs, int src_dtype, int64_t n_src_rows, int64_t layers,
                   int64_t hidden, const int64_t* src_ids, const void* src_mask, int mask_elem,
                   const int64_t* src_pos, const int64_t* src_start, const int64_t* out_start,
                   int64_t n_docs, int64_t max_len, int shift, void* out_aux, void* out_last,
                   int64_t* out_ids, void* out_mask, int64_t* out_pos, int64_t* out_doc,
                   void* stream);

/* Masked mean and acceptance chain of one TTT step over `rows` aligned rows:
 *   out[0] = weight * sum_r loss[r] * m_r / (sum_r m_r + 1e-5)
 *            (loss_function, losses/utils.py:269-304, with the exp_loss_decay
 *            weight gamma**step, losses/utils.py:51-61, passed as `weight`)
 *   out[1] = full_correct = out[3] = cond_correct
 *            = #{r : m_r != 0 and prev_r and pred_r == tgt_r}
 *   out[2] = full_total = #{r : m_r != 0}
 *   out[4] = cond_total = #{r : prev_r}  counted BEFORE the update
 *   out[5] = sum_r m_r
 *   prev_correct[r] <- prev_correct[r] and (pred_r == tgt_r), in place
 *   row_weight[r]   = weight * m_r / (sum m + 1e-5)   (d out[0] / d loss[r])
 * Replaces the reduction of loss_function and compute_accuracy_single_step
 * (models/metrics.py:6-36) as called from compute_metrics
 * (models/eagle3/metrics.py:86-117).  `mask` / `prev_correct` may be NULL
 * (all ones / not tracked: then cond_total = rows).  Counts are exact
 * integers stored as fp32 (rows < 2^24).  Deterministic. */
int spx_ttt_step_reduce(const float* loss, const int32_t* argmax_draft,
                        const int32_t* argmax_target, const void* mask,
                        int mask_kind, void* prev_correct, int prev_kind,
                        int64_t rows, float weight, float* out,
                        float* row_weight, void* stream);

/* spx_ttt_step_reduce for a step whose acceptance chain was already done row by row by
 * spx_vocab_loss_step_fwd: the masked mean and row_weight as there, out[1] = out[3] =
 * counts[0], out[2] = counts[1], out[4] = counts[2], out[5] = sum of the mask. */
int spx_ttt_step_mean(const float* loss, const void* mask, int mask_kind, int64_t rows,
                      float weight, const int32_t* counts, float* out, float* row_weight,
                      void* stream);

/* Weighted masked mean and per-slot acceptance counts of a DFlash block batch:
 *   out[0] = sum_r loss[r] m_r w_r / (sum m + 1e-5),  out[1] = sum m
 *   correct[s], total[s]  (s < block_size): matches / rows with m_r != 0 at
 *   slot s = r % block_size   (compute_accuracy_multi_step, models/metrics.py:39-69)
 *   row_weight[r] = m_r w_r / (sum m + 1e-5)
 * `pos_weight` (fp32 [rows]) is the per-row weight: dflash_loss_decay
 * (losses/utils.py:17-48) or the D-PACE weight (losses/utils.py:64-112);
 * NULL = 1.  Replaces the reduction part of models/dflash/metrics.py:20-108. */
int spx_block_reduce(const float* loss, const int32_t* argmax_draft,
                     const int32_t* argmax_target, const void* mask,
                     int mask_kind, const float* pos_weight, int64_t rows,
                     int32_t block_size, float* out, float* correct,
                     float* total, float* row_weight, void* stream);

/* ---------------------------------------------------------------- TTT attention
 * row_lo[i] = lowest context key visible to query i: the interval form
 * row_lo[i] <= c <= i of the step-0 part of create_combined_mask_mod
 * (models/eagle3/attention.py:11-34) for run-contiguous document ids (what
 * CollateFn emits, train/data.py:323-393): start of i's document, raised to
 * i - W + 1 under a sliding window W (sliding_window <= 0: none), and i itself
 * for padding rows (document id -1).  Replaces the dense [T, T] mask that
 * create_block_mask materialises (models/eagle3/core.py:149-162). */
int spx_ttt_row_lo(const void* document_ids, int doc_kind, int64_t T,
                   int64_t sliding_window, int32_t* row_lo, void* stream);

/* bytes of caller-owned scratch the attention entry points need */
int64_t spx_ttt_attn_workspace_bytes(int64_t T, int32_t Hq, int32_t Hkv,
                                     int32_t D, int32_t backward);

/* out[i, h, :] = softmax_c(scaling * q[h, i] . k[h / (Hq/Hkv), c]) v[..]  over the
 * keys of TTT step `ttt_step` (0-based): context keys row_lo[i] <= c <= i of
 * the first T rows of k/v, plus the rows j*T + i for j = 1..ttt_step (the
 * diagonals that extend_mask_for_draft_tokens appends,
 * models/eagle3/attention.py:37-132).  Replaces flex_attention_forward
 * (models/attention.py:20-66) for the EAGLE3 mask.
 *   q   bf16 [Hq, T, D]  (head stride q_head_stride elements, rows contiguous)
 *   k,v bf16 [Hkv, (ttt_step+1)*T, D]  (the cache layout of DynamicCache)
 *   out bf16 [T, Hq, D];  lse f32 [Hq, T]: log2-domain row log-sum-exp, opaque,
 *   consumed by spx_ttt_attn_bwd.   D in {64, 128, 256}. */
int spx_ttt_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                     int64_t k_head_stride, const void* v, int64_t v_head_stride,
                     const int32_t* row_lo, int64_t T, int32_t ttt_step,
                     int32_t Hq, int32_t Hkv, int32_t D, float scaling,
                     void* out, float* lse, void* workspace,
                     int64_t workspace_bytes, void* stream);

/* spx_ttt_attn_fwd without a workspace argument, for callers that cannot allocate one:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has
 * no counterpart in the reference.  The forward's only scratch, the key-contiguous copy
 * V^T [Hkv, D, round_up(T, 128)] bf16, lives in a static device array of
 * spx_ttt_attn_fwd_static_max_bytes() = 16 MiB inside the library (each GPU the library runs
 * on holds it until the process ends); shapes with Hkv * D * round_up(T, 128) * 2 bytes above
 * that are rejected with status 1 (use spx_ttt_attn_fwd).  Neither this call nor anything it
 * launches allocates or frees memory.  Results are bit-identical to spx_ttt_attn_fwd.  All calls
 * on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two
 * host threads) race on it; calls ordered on one stream do not.  Nothing has to be cleared
 * between calls: each call rewrites every byte of the array it later reads.
 * The FIRST call on a device for a given head_dim does set-up work that is not allowed while a
 * stream is being captured (it looks up the array's address, which may load the code object, and
 * raises the kernel's dynamic-LDS limit): make one call per device and head_dim outside capture
 * before capturing; every later call only launches kernels. */
int64_t spx_ttt_attn_fwd_static_max_bytes(void);
int spx_ttt_attn_fwd_static(const void* q, int64_t q_head_stride, const void* k,
                            int64_t k_head_stride, const void* v, int64_t v_head_stride,
                            const int32_t* row_lo, int64_t T, int32_t ttt_step,
                            int32_t Hq, int32_t Hkv, int32_t D, float scaling,
                            void* out, float* lse, void* stream);

/* Gradients of spx_ttt_attn_fwd.  dout bf16 [T, Hq, D] (the layout of `out`),
 * lse as written by the forward.  dq bf16 [Hq, T, D]; dk, dv bf16
 * [Hkv, (ttt_step+1)*T, D]: every row is written (context rows by the tiled
 * kernels, the diagonal rows j*T + i by a per-position kernel; no atomics, so
 * the result is deterministic).  Replaces the autograd of flex_attention at
 * the call site models/attention.py:55-63. */
int spx_ttt_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                     int64_t k_head_stride, const void* v, int64_t v_head_stride,
                     const void* out, const void* dout, const float* lse,
                     const int32_t* row_lo, int64_t T, int32_t ttt_step,
                     int32_t Hq, int32_t Hkv, int32_t D, float scaling, void* dq,
                     int64_t dq_head_stride, void* dk, int64_t dk_head_stride,
                     void* dv, int64_t dv_head_stride, void* workspace,
                     int64_t workspace_bytes, void* stream);

/* The same, ADDING to what dk and dv hold (dq is written): dk = bf16(float(dk) + this call's
 * gradient), one rounding per call.  The K / V rows of one TTT step are keys of every later step
 * (DynamicCache.update, models/eagle3/core.py:283-300), so their gradient is a sum over the steps'
 * backwards, which the reference's autograd forms with one add per tensor and step.  A caller that
 * owns one [Hkv, steps*T, D] gradient buffer per layer runs the last step's backward with
 * spx_ttt_attn_bwd (every row of its (ttt_step+1)*T written) and the earlier steps' with this
 * entry point, in descending step order on one stream. */
int spx_ttt_attn_bwd_accumulate(const void* q, int64_t q_head_stride, const void* k,
                                int64_t k_head_stride, const void* v, int64_t v_head_stride,
                                const void* out, const void* dout, const float* lse,
                                const int32_t* row_lo, int64_t T, int32_t ttt_step,
                                int32_t Hq, int32_t Hkv, int32_t D, float scaling, void* dq,
                                int64_t dq_head_stride, void* dk, int64_t dk_head_stride,
                                void* dv, int64_t dv_head_stride, void* workspace,
                                int64_t workspace_bytes, void* stream);

/* Attention with one interval of visible keys per query: out[i, h, :] = softmax over the keys
 * row_lo[i] <= c < row_hi[i] (out of T; an empty interval gives a zero row).  This is the mask
 * transformers' create_causal_mask builds from a 2-D padding mask -- key j visible to query i iff
 * j <= i and attention_mask[j] -- when the non-padding positions of a row are contiguous, which is
 * how the MTP forward is called with `attention_mask` (models/mtp/core.py:180-186, 119).  Layouts,
 * lse, workspace sizes (spx_ttt_attn_workspace_bytes) and determinism as for spx_ttt_attn_fwd /
 * spx_ttt_attn_bwd at ttt_step 0. */
int spx_span_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                      int64_t k_head_stride, const void* v, int64_t v_head_stride,
                      const int32_t* row_lo, const int32_t* row_hi, int64_t T,
                      int32_t Hq, int32_t Hkv, int32_t D, float scaling,
                      void* out, float* lse, void* workspace,
                      int64_t workspace_bytes, void* stream);
int spx_span_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                      int64_t k_head_stride, const void* v, int64_t v_head_stride,
                      const void* out, const void* dout, const float* lse,
                      const int32_t* row_lo, const int32_t* row_hi, int64_t T,
                      int32_t Hq, int32_t Hkv, int32_t D, float scaling, void* dq,
                      int64_t dq_head_stride, void* dk, int64_t dk_head_stride,
                      void* dv, int64_t dv_head_stride, void* workspace,
                      int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------- DFlash attention
 * Per-row key intervals of the anchored-block mask, create_anchor_block_mask_mod
 * (models/dflash/attention.py:7-100), for run-contiguous document ids.  Row
 * r = j*block_size + s belongs to anchor j (position a_j):
 *   context keys  ctx_lo[r] <= c < ctx_hi[r]:  ctx_hi = a_j, ctx_lo = start of
 *     a_j's document, raised to a_j - W under a sliding window W (<= 0: none);
 *     empty when a_j sits on a padding position;
 *   block keys (rows T + c of k/v)  blk_lo[r] <= c < blk_hi[r]:  the rows of the
 *     query's own block, all of them, or only c <= r when causal_block != 0
 *     (a sliding-window layer without sliding_window_non_causal).
 * run_start_scratch: int32 [T] scratch.  Replaces the compiled create_block_mask
 * of models/dflash/core.py:273-328. */
int spx_dflash_row_ranges(const void* document_ids, int doc_kind, int64_t T,
                          const void* anchors, int anchor_kind, int64_t n_anchors,
                          int32_t block_size, int64_t sliding_window,
                          int32_t causal_block, int32_t* ctx_lo, int32_t* ctx_hi,
                          int32_t* blk_lo, int32_t* blk_hi,
                          int32_t* run_start_scratch, void* stream);

int64_t spx_dflash_attn_workspace_bytes(int64_t T, int64_t NQ, int32_t Hq,
                                        int32_t Hkv, int32_t D, int32_t backward);

/* Anchored-block attention: q bf16 [Hq, NQ, D] (NQ = n_anchors * block_size mask
 * tokens), k/v bf16 [Hkv, T + NQ, D] = context keys followed by the mask-token
 * keys (the concatenation Qwen3DFlashAttention builds,
 * models/dflash/model_definitions.py:97-155); out bf16 [NQ, Hq, D]; lse f32
 * [Hq, NQ] (opaque).  Replaces flex_attention_forward (models/attention.py:20-66)
 * for the DFlash mask. */
int spx_dflash_attn_fwd(const void* q, int64_t q_head_stride, const void* k,
                        int64_t k_head_stride, const void* v, int64_t v_head_stride,
                        const int32_t* ctx_lo, const int32_t* ctx_hi,
                        const int32_t* blk_lo, const int32_t* blk_hi, int64_t T,
                        int64_t NQ, int32_t Hq, int32_t Hkv, int32_t D,
                        float scaling, void* out, float* lse, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* Gradients of spx_dflash_attn_fwd: dq [Hq, NQ, D], dk / dv [Hkv, T + NQ, D],
 * every row written, deterministic. */
int spx_dflash_attn_bwd(const void* q, int64_t q_head_stride, const void* k,
                        int64_t k_head_stride, const void* v, int64_t v_head_stride,
                        const void* out, const void* dout, const float* lse,
                        const int32_t* ctx_lo, const int32_t* ctx_hi,
                        const int32_t* blk_lo, const int32_t* blk_hi, int64_t T,
                        int64_t NQ, int32_t Hq, int32_t Hkv, int32_t D,
                        float scaling, void* dq, int64_t dq_head_stride, void* dk,
                        int64_t dk_head_stride, void* dv, int64_t dv_head_stride,
                        void* workspace, int64_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------- layer glue
 * RMSNorm with the rounding points of the HF blocks the reference builds on
 * (LlamaRMSNorm / Qwen3RMSNorm as used in models/eagle3/model_definitions.py:70-85,
 * models/eagle3/core.py:236-253,302-306, models/dflash/model_definitions.py:97-155):
 * y = weight * bf16(x * rsqrt(mean(x^2) + eps)), bf16 in/out, rstd f32 [rows]
 * saved for the backward (may be NULL). */
int spx_rmsnorm_fwd(const void* x, int64_t ld_x, const void* weight, void* y,
                    int64_t ld_y, float* rstd, int64_t rows, int64_t H, float eps,
                    void* stream);
/* number of partial-sum slots the backward needs: dw_scratch holds slots * H floats */
int64_t spx_rmsnorm_bwd_slots(int64_t rows, int64_t H);
/* dx (may be NULL when only dweight is wanted) and (optionally, dweight != NULL)
 * dweight = sum_rows dy * xhat, reduced in a fixed order (deterministic). */
int spx_rmsnorm_bwd(const void* x, int64_t ld_x, const void* weight, const void* dy,
                    int64_t ld_dy, const float* rstd, void* dx, int64_t ld_dx,
                    void* dweight, float* dw_scratch, int64_t rows, int64_t H,
                    void* stream);
/* The residual add in front of a norm fused into it: sum = bf16(a + b) (written, it is
 * the residual stream) and y = rmsnorm(sum).  Replaces `hidden_states = residual +
 * hidden_states` followed by the next RMSNorm in the decoder layer
 * (models/eagle3/model_definitions.py:96-110 and the HF LlamaDecoderLayer it patches;
 * models/eagle3/core.py:302-306 for the final norm). */
int spx_add_rmsnorm_fwd(const void* a, int64_t ld_a, const void* b, int64_t ld_b, void* sum,
                        int64_t ld_sum, const void* weight, void* y, int64_t ld_y,
                        float* rstd, int64_t rows, int64_t H, float eps, void* stream);
/* Its backward: dx = dres + rmsnorm_bwd(dy) in one rounding, where dres (may be NULL)
 * is the gradient reaching `sum` along the residual stream; x is the saved `sum`.
 * dx is the gradient of both a and b. */
int spx_add_rmsnorm_bwd(const void* x, int64_t ld_x, const void* weight, const void* dy,
                        int64_t ld_dy, const void* dres, int64_t ld_dres, const float* rstd,
                        void* dx, int64_t ld_dx, void* dweight, float* dw_scratch,
                        int64_t rows, int64_t H, void* stream);
/* The backward of either norm for a gain that is applied several times in one forward (once per
 * TTT step: models/eagle3/core.py:286-306): dx as above (dres may be NULL), while the gain's
 * gradient stays as partial sums in dw_scratch (spx_rmsnorm_bwd_slots(rows, H) * H floats) --
 * written when accumulate == 0, added to when != 0 (every use with the same rows and H) -- until
 * spx_rmsnorm_dweight reduces them once, in a fixed order, to dweight (bf16 [H]).  The sum over the
 * uses is then formed in fp32 with one rounding, where autograd adds rounded per-use gradients. */
int spx_rmsnorm_bwd_partial(const void* x, int64_t ld_x, const void* weight, const void* dy,
                            int64_t ld_dy, const void* dres, int64_t ld_dres,
                            const float* rstd, void* dx, int64_t ld_dx, float* dw_scratch,
                            int32_t accumulate, int64_t rows, int64_t H, void* stream);
int spx_rmsnorm_dweight(const float* dw_scratch, int64_t slots, int64_t H, void* dweight,
                        void* stream);

/* Rotary embedding fused with the head-major relayout that precedes attention
 * (apply_rotary_pos_emb + the view/transpose of LlamaAttention.forward; for
 * DFlash models/dflash/model_definitions.py:29-45):
 *   inverse == 0: out[h, t, :] = rope(x[t, h*D : (h+1)*D], position_ids[t] + position_offset)
 *   inverse != 0: out[t, h*D : (h+1)*D] = rope^T(x[h, t, :], ...)   (its backward)
 * rotate == 0 only relayouts (V).  inv_freq: f32 [D/2].  Half-split rotation,
 * cos/sin evaluated in fp32 and rounded to bf16 like the HF rotary module.
 * The stride argument of the head-major side (ld_out when inverse == 0, ld_x otherwise) is
 * its HEAD stride in elements, 0 meaning T * D: the head-major tensor may be a window of a
 * longer K/V cache [heads, steps * T, D] (DynamicCache.update without the copy). */
int spx_rope_relayout(const void* x, int64_t ld_x, const int64_t* position_ids,
                      const float* inv_freq, void* out, int64_t ld_out, int64_t T,
                      int32_t heads, int32_t D, int32_t rotate, int32_t inverse,
                      int64_t position_offset, void* stream);

/* The same with the two things the hybrid MTP flavours need (their layers are the library's
 * Qwen3NextDecoderLayer / Qwen3_5DecoderLayer / Qwen3_5MoeDecoderLayer, wrapped at
 * models/mtp/model_definitions.py:159-205): the token-major side has a head stride of its own
 * (x_head_stride elements; the widened q projection holds [query | gate] per head, 2 D apart), and
 * only the first rotary_dim elements of every head are rotated (pairs i, i + rotary_dim / 2; the
 * rest is copied), rotary_dim a multiple of 16, inv_freq f32 [rotary_dim / 2].  table_scale
 * multiplies cos and sin before they are rounded: the attention factor of the yarn frequency
 * scaling (`cos = emb.cos() * self.attention_scaling` in the library's rotary modules), 1 otherwise. */
int spx_rope_relayout_partial(const void* x, int64_t ld_x, int32_t x_head_stride,
                              const int64_t* position_ids, const float* inv_freq, void* out,
                              int64_t ld_out, int64_t T, int32_t heads, int32_t D,
                              int32_t rotary_dim, int32_t rotate, int32_t inverse,
                              int64_t position_offset, float table_scale, void* stream);

/* Output gate of the gated attention (`attn_output * torch.sigmoid(gate)` of Qwen3NextAttention,
 * reached through models/mtp/model_definitions.py:159-205): y = bf16(o * bf16(sigmoid(gate))) on
 * [rows, heads, D] bf16 tensors; o, y, dy, d_o have contiguous heads and a row stride, the gate
 * and its gradient a row stride and a head stride (they are the second halves of the 2 D columns
 * per head of the q projection and of its output gradient).  Backward: d_o = dy * sig,
 * dgate = dy * o * sig * (1 - sig). */
int spx_sigmoid_gate_fwd(const void* o, int64_t ld_o, const void* gate, int64_t ld_gate,
                         int32_t gate_head_stride, void* y, int64_t ld_y, int64_t rows,
                         int32_t heads, int32_t D, void* stream);
int spx_sigmoid_gate_bwd(const void* o, int64_t ld_o, const void* gate, int64_t ld_gate,
                         int32_t gate_head_stride, const void* dy, int64_t ld_dy, void* d_o,
                         int64_t ld_do, void* dgate, int64_t ld_dgate, int32_t dgate_head_stride,
                         int64_t rows, int32_t heads, int32_t D, void* stream);

/* out = bf16(silu(gate)) * up  (LlamaMLP / Qwen3MLP act_fn(gate_proj(x)) * up_proj(x)),
 * bf16; and its backward.  rows x F elements per tensor, each with its own row stride, so
 * that gate and up can be the two column halves of one merged gate/up projection. */
int spx_swiglu_rows_fwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                        void* out, int64_t ld_out, int64_t rows, int64_t F, void* stream);
int spx_swiglu_rows_bwd(const void* gate, int64_t ld_gate, const void* up, int64_t ld_up,
                        const void* dout, int64_t ld_dout, void* dgate, int64_t ld_dgate,
                        void* dup, int64_t ld_dup, int64_t rows, int64_t F, void* stream);
/* the same on contiguous tensors of n elements */
int spx_swiglu_fwd(const void* gate, const void* up, void* out, int64_t n, void* stream);
int spx_swiglu_bwd(const void* gate, const void* up, const void* dout, void* dgate,
                   void* dup, int64_t n, void* stream);

/* ---------------------------------------------------------------- GEMM
 * c[M, N] = a[M, K] * b[N, K]^T, bf16 inputs, fp32 accumulation, bf16 output:
 * the product of torch.nn.Linear (no bias).  Replaces the fc Linear
 * (models/eagle3/core.py:76,244), the lm_head and verifier_lm_head Linears
 * (model.py:66-69; call sites models/eagle3/core.py:251-253,302-306) and, with
 * b = the transposed weight, the input-gradient product of their backward.
 * lda/ldb/ldc are row strides in elements; K, lda, ldb multiples of 8; 256 rows
 * of an operand span less than 2 GiB (the operands themselves may be larger). */
int spx_gemm_bf16_nt(const void* a, int64_t lda, const void* b, int64_t ldb,
                     void* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                     void* stream);

/* spx_gemm_bf16_nt for products whose number of 256 x 256 output tiles leaves the last round of
 * workgroups mostly empty (384 tiles on 256 compute units: the second round is half empty and
 * takes as long as a full one).  The tiles of that last round -- when they are at most half a
 * round -- are cut along the contraction into up to max_parts parts (fp32 partials in the
 * workspace, added in a fixed order by a second small kernel: results do not depend on timing);
 * every other tile is computed and stored exactly as by spx_gemm_bf16_nt, and so is every tile
 * when the last round is more than half full.  workspace: spx_gemm_tail_workspace_bytes()
 * bytes, 16-byte aligned, caller owned.  No counterpart in the reference (its Linears run on
 * the vendor library, which picks another tile shape for such products). */
int64_t spx_gemm_tail_workspace_bytes(void);
int spx_gemm_bf16_nt_tail(const void* a, int64_t lda, const void* b, int64_t ldb,
                          void* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                          int32_t max_parts, void* workspace, int64_t workspace_bytes,
                          void* stream);

/* spx_gemm_bf16_nt whose epilogue also yields, per row m of c, the soft-max statistics of that
 * row AS ROUNDED TO bf16: lse[m] = log sum_n exp(c[m, n]) (natural logarithm, fp32) and
 * argmax[m] = the first n that attains max_n c[m, n] (-0 and +0 compare equal, as torch.argmax
 * has it).  Either of lse and argmax may be null (not both): what is not asked for is not
 * computed.  These are what the loss kernels otherwise compute by streaming c again:
 * with them a cross-entropy against arg-max targets (losses/eager.py ce_loss; the eager
 * reference takes argmax of the full target logits, models/eagle3/metrics.py:100-117) never
 * needs the target logits in memory, and the full-vocabulary cross-entropy of MTP
 * (models/mtp/core.py:190-226) needs lse[m] and one element of row m only.  This is the
 * forward half of "lm_head + loss in one pass": c MAY BE NULL, then the product is reduced to
 * its statistics and never written.  workspace: spx_gemm_stats_workspace_bytes(M, N) bytes
 * (per-tile partial statistics, 12 bytes per row and 256 columns), 4-byte aligned, caller owned. */
int64_t spx_gemm_stats_workspace_bytes(int64_t M, int64_t N);
int spx_gemm_bf16_nt_stats(const void* a, int64_t lda, const void* b, int64_t ldb,
                           void* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                           float* lse, int32_t* argmax, void* workspace,
                           int64_t workspace_bytes, void* stream);

/* The same product with the number of rows of a (and c) that count read from device
 * memory at run time: rows >= min(M, *m_live) are neither read nor written.  For an
 * operand whose producer packs its live rows to the front (spx_label_ce_bwd_packed:
 * positions with an ignored label have a zero gradient row, models/mtp/core.py:204-216)
 * without the host learning how many there are.  No counterpart in the reference. */
int spx_gemm_bf16_nt_rows(const void* a, int64_t lda, const void* b, int64_t ldb,
                          void* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                          const int32_t* m_live, void* stream);

/* spx_gemm_bf16_nt_rows with the contraction cut into up to max_parts (1 .. 8) parts when the tiles of
 * the rows that count leave compute units idle: the product of 2860 live rows by a 4096-column weight is
 * 192 tiles of 256 x 256 on 256 compute units, one round of a whole contraction; cut in four it is three
 * rounds of a quarter.  The kernel chooses the number of parts from the row count it reads on the device
 * (the count that needs the fewest rounds, if that saves a tenth or more; else one part and the direct
 * bf16 store of spx_gemm_bf16_nt_rows); every part leaves an fp32 partial in `workspace`
 * (spx_gemm_split_workspace_bytes(M, N, max_parts) = max_parts * M * N * 4 bytes, 16-byte aligned) and a
 * second kernel adds the parts in their order, so the result does not depend on scheduling.  N and ldc
 * multiples of 8, c 16-byte aligned; m_live may be NULL (all M rows count).  Used for the lm_head
 * input-gradient product of the frozen head (model.py:66-69 is the Linear whose backward this is).
 * No counterpart in the reference. */
int64_t spx_gemm_split_workspace_bytes(int64_t M, int64_t N, int32_t max_parts);
int spx_gemm_bf16_nt_rows_split(const void* a, int64_t lda, const void* b, int64_t ldb,
                                void* c, int64_t ldc, int64_t M, int64_t N, int64_t K,
                                const int32_t* m_live, int32_t max_parts, void* workspace,
                                int64_t workspace_bytes, void* stream);

/* The two ends of a packed-rows product (spx_*_bwd_packed -> spx_gemm_bf16_nt_rows).
 * spx_pack_row_map: row_map[r] = number of live rows before r if row r is live
 * (row_grad[r] != 0 and, when labels is not NULL, labels[r] != ignore_index), else -1;
 * *count = number of live rows (device memory: the host never reads it).
 * spx_unpack_rows (bf16): out[r, :] = packed[row_map[r], :] for live rows, zeros for
 * the others and for rows <= r < total_rows.  No counterpart in the reference. */
int spx_pack_row_map(const float* row_grad, const int64_t* labels, int64_t ignore_index,
                     int64_t rows, int32_t* row_map, int32_t* count, void* stream);
int spx_unpack_rows(const void* packed, int64_t ld_packed, const int32_t* row_map,
                    int64_t rows, int64_t total_rows, int64_t cols, void* out,
                    int64_t ld_out, void* stream);
/* The same with every live row multiplied by row_scale[r] (f32 [rows]) on its way: the row
 * weights of a product whose packed operand was made for unit weights
 * (spx_vocab_loss_step_fwd_grad). */
int spx_unpack_rows_scaled(const void* packed, int64_t ld_packed, const int32_t* row_map,
                           const float* row_scale, int64_t rows, int64_t total_rows,
                           int64_t cols, void* out, int64_t ld_out, void* stream);

/* c[M, N] (+)= a[T, M]^T * b[T, N], bf16 inputs, fp32 accumulation, bf16 output:
 * the weight-gradient product of the backward of torch.nn.Linear (dW = dY^T X)
 * for every Linear of the draft layers (models/eagle3/core.py:76,244 and the
 * q/k/v/o/gate/up/down projections of the decoder layer, model_definitions.py).
 * accumulate != 0 adds the product to what c holds (one rounding to bf16 of
 * old + product): the weights are applied once per TTT step and their gradients
 * sum over the steps (models/eagle3/core.py:289-345).  M, N, lda, ldb multiples
 * of 8; a and b 16-byte aligned; each operand spans less than 2 GiB. */
int spx_gemm_bf16_tn(const void* a, int64_t lda, const void* b, int64_t ldb,
                     void* c, int64_t ldc, int64_t M, int64_t N, int64_t T,
                     int accumulate, void* stream);

/* The same product with an fp32 result c[M, N] (ldc in floats): with accumulate != 0
 * the weight gradient sums over the TTT steps in fp32 with no rounding between
 * them, which is what autograd's accumulation into an fp32 master weight's .grad
 * does in the reference's trainer (train/trainer.py:459-465 runs the model under
 * bf16 autocast over fp32 parameters). */
int spx_gemm_bf16_tn_f32(const void* a, int64_t lda, const void* b, int64_t ldb,
                         void* c, int64_t ldc, int64_t M, int64_t N, int64_t T,
                         int accumulate, void* stream);

/* ---------------------------------------------------------------- sparse MoE block
 * The expert products of the MoE MLP of the hybrid MTP flavours (Qwen3NextSparseMoeBlock /
 * Qwen3NextExperts of the library, reached through models/mtp/model_definitions.py:159-205).
 * The library loops over the experts that were hit, gathering each one's tokens; here the
 * (token, slot) pairs are sorted by expert once and every product runs over all experts in one
 * launch.  group_offsets: int32 [groups + 1] on the device, non-decreasing from 0 to at most
 * `rows`; group e owns the sorted rows [group_offsets[e], group_offsets[e + 1]).  The host never
 * reads the offsets.
 *
 * spx_gemm_bf16_nt_grouped: c[r, :] = a[r, :] * b_e^T for the rows r of group e, b_e = b +
 * e * b_group_stride ([N, K], row stride ldb).  The workspace (spx_gemm_grouped_workspace_bytes,
 * 4-byte aligned) holds the tile table the launch builds on the device.  Same operand rules as
 * spx_gemm_bf16_nt.
 * spx_gemm_bf16_tn_grouped: c_e[M, N] (+)= a[rows of e, :M]^T * b[rows of e, :N], c_e = c +
 * e * c_group_stride elements; out_f32 selects an fp32 c; without `accumulate` an empty group
 * gets zeros.  Same operand rules as spx_gemm_bf16_tn. */
int64_t spx_gemm_grouped_workspace_bytes(int64_t rows, int64_t groups);
int spx_gemm_bf16_nt_grouped(const void* a, int64_t lda, const void* b, int64_t ldb,
                             int64_t b_group_stride, void* c, int64_t ldc, int64_t rows,
                             int64_t N, int64_t K, const int32_t* group_offsets, int64_t groups,
                             void* workspace, int64_t workspace_bytes, void* stream);
int spx_gemm_bf16_tn_grouped(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                             int64_t ldc, int64_t c_group_stride, int64_t M, int64_t N,
                             int64_t rows, const int32_t* group_offsets, int64_t groups,
                             int out_f32, int accumulate, void* stream);
/* The same over `segments` segments of `segment_rows` rows each, one below the other in a and b
 * (the expert-sorted rows of the K prediction steps of an MTP forward, models/mtp/core.py:190-226
 * applies the layer once per step): group_offsets is int32 [segments][groups + 1], each row
 * relative to its segment, and c_e (+)= sum over the segments of the group's product.  The sum
 * over the steps happens in the accumulators; c is written once.  A segment whose row of offsets
 * is all zero contributes nothing. */
int spx_gemm_bf16_tn_grouped_multi(const void* a, int64_t lda, const void* b, int64_t ldb, void* c,
                                   int64_t ldc, int64_t c_group_stride, int64_t M, int64_t N,
                                   int64_t segment_rows, int64_t segments,
                                   const int32_t* group_offsets, int64_t groups, int out_f32,
                                   int accumulate, void* stream);

/* out[b][c][r] = in[b][r][c] for `batches` bf16 matrices of R x C (multiples of 8), row strides
 * ld_in / ld_out and batch strides in elements: the transposed copies the input-gradient
 * products need of a weight stack (a product against W needs W^T in this library's NT form; the
 * reference's autograd gets it from the BLAS library's NN form).  No counterpart in the
 * reference. */
int spx_transpose_bf16(const void* in, int64_t ld_in, int64_t batch_stride_in, void* out,
                       int64_t ld_out, int64_t batch_stride_out, int64_t R, int64_t C,
                       int64_t batches, void* stream);

/* Row movement between the token order [tokens, H] and the expert-sorted order [rows, H] (bf16;
 * index_select / index_add_ of Qwen3NextExperts.forward and their backward):
 *   spx_moe_gather_rows:  out[p] = scale[p] * x[src_row[p]]   (scale f32 [rows] or NULL; an index
 *                         outside [0, src_rows) gives a zero row)
 *   spx_moe_combine_rows: out[t] = sum_j weight[t, j] * sorted[pos[t, j]], j = 0 .. k-1 in that
 *                         order in fp32, one rounding (weight f32 [tokens, k] or NULL = ones)
 *   spx_moe_pair_dot:     out[t, j] = <a[t], sorted[pos[t, j]]> in fp32 (the gradient of the
 *                         routing weights). */
int spx_moe_gather_rows(const void* x, int64_t ld_x, int64_t src_rows, const int32_t* src_row,
                        const float* scale, void* out, int64_t ld_out, int64_t rows, int64_t H,
                        void* stream);
int spx_moe_combine_rows(const void* sorted, int64_t ld_sorted, int64_t sorted_rows,
                         const int32_t* pos, const float* weight, void* out, int64_t ld_out,
                         int64_t tokens, int32_t k, int64_t H, void* stream);
int spx_moe_pair_dot(const void* a, int64_t ld_a, const void* sorted, int64_t ld_sorted,
                     int64_t sorted_rows, const int32_t* pos, float* out, int64_t tokens,
                     int32_t k, int64_t H, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPX_H */

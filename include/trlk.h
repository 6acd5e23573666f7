/*
 * trlk -- C ABI of the MI355X (gfx950) kernels for TRL's per-token log-probability,
 * entropy and policy-loss path.
 *
 * Conventions (all entry points):
 *   - every pointer named `d_*` is DEVICE memory owned by the caller; the library never
 *     allocates, frees or keeps a pointer after the call returns;
 *   - calls only enqueue work on `stream` (a hipStream_t passed as void*; NULL = the
 *     default stream) and never synchronise the host;
 *   - return value: 0 = enqueued; negative = argument error found on the host before
 *     anything was launched (see trlk_status, text in trlk_last_error()); positive =
 *     the hipError_t of a failed launch;
 *   - "rows" are token positions.  A logits operand is a strided 3-D view
 *     [n_seq, rows_per_seq, vocab] whose last axis is contiguous: element (b, t, v) is at
 *     `base + b*seq_stride + t*row_stride + v` (strides in ELEMENTS).  Per-row operands
 *     (indices, log-probs, masks, gradients) are dense row-major [n_seq*rows_per_seq(, K)].
 *
 * The reference has no native code; each entry point names the Python lines whose
 * arithmetic it replaces (paths relative to the reference tree).
 */
#ifndef TRLK_H
#define TRLK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRLK_VERSION 2

typedef void* trlk_stream_t; /* hipStream_t */

enum trlk_dtype { TRLK_F32 = 0, TRLK_BF16 = 1, TRLK_F16 = 2 };

enum trlk_status {
    TRLK_OK = 0,
    TRLK_ERR_NULL_POINTER = -1,
    TRLK_ERR_BAD_SHAPE = -2,
    TRLK_ERR_BAD_DTYPE = -3,
    TRLK_ERR_BAD_STRIDE = -4,
    TRLK_ERR_BAD_VALUE = -5,
    TRLK_ERR_WORKSPACE = -6,
    TRLK_ERR_UNSUPPORTED = -7
};

/* loss normalisations of GRPOTrainer._compute_loss (trl/trainer/grpo_trainer.py:3124-3142) */
enum trlk_grpo_loss_type { TRLK_GRPO = 0, TRLK_BNPO = 1, TRLK_DR_GRPO = 2, TRLK_DAPO = 3, TRLK_LUSPO = 4 };

/* per-token policy term of the GRPO family (trl/trainer/grpo_trainer.py:3080-3107); c = importance ratio, A = advantage
 *   CLIP:          -min(min(c, delta) * A, clamp(c, 1-eps_low, 1+eps_high) * A)     grpo, bnpo, dr_grpo, dapo, luspo
 *   CISPO:         -min(c, eps_high).detach() * A * logp                            cispo
 *   SAPO:          -sigmoid(tau * (c - 1)) * 4 / tau * A, tau = A > 0 ? pos : neg    sapo
 *   WEIGHTED_LOGP: -coef[b] * A * logp with a given, detached per-sequence coef      vespo (coef = gamma weights) */
enum trlk_grpo_policy_term { TRLK_TERM_CLIP = 0, TRLK_TERM_CISPO = 1, TRLK_TERM_SAPO = 2, TRLK_TERM_WEIGHTED_LOGP = 3 };

/* scale_rewards modes (trl/trainer/grpo_trainer.py:2687-2707) */
enum trlk_scale_rewards { TRLK_SCALE_GROUP = 0, TRLK_SCALE_BATCH = 1, TRLK_SCALE_NONE = 2 };

/* bits of the int32 word the kernels OR into `d_error_flag` */
#define TRLK_FLAG_INDEX_OUT_OF_RANGE 1

int trlk_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char* trlk_last_error(void);

/* ---------------------------------------------------------------------------------------
 * K1  log-prob + entropy forward, one streaming pass over the logits.
 * Replaces selective_log_softmax (trl/trainer/utils.py:479-523), entropy_from_logits
 * (utils.py:526-560) and the temperature division in front of them
 * (trl/trainer/grpo_trainer.py:1519): with z = logits / temperature,
 *   out_logp[r, k] = z[r, index[r, k]] - logsumexp(z[r, :])
 *   out_entropy[r] = logsumexp(z[r, :]) - sum_v softmax(z[r])_v * z[r, v]
 *   out_lse[r]     = logsumexp(z[r, :])            (the only state the backward needs)
 * All arithmetic is fp32 whatever `dtype` is; outputs are fp32.
 * d_index: int64 [rows, n_index].  d_row_mask (optional, uint8 [rows]): rows whose mask is 0
 * are not read and get 0 in every output.  d_out_entropy / d_out_lse / d_out_row_stats /
 * d_error_flag may be NULL.
 * d_out_row_stats (optional, fp32 [rows, 4]) takes what DPOTrainer._compute_loss derives from
 * three more passes over the logits (trl/trainer/dpo_trainer.py:1563-1574 WPO weights, :1605-1618
 * logits means, :1620-1631 token accuracy):
 *   [0] mean_v logits[r, v]                       (raw logits, not divided by the temperature)
 *   [1] log sum_v softmax(z[r])_v^2 = logsumexp(2 z) - 2 logsumexp(z) if row_stats_sum_p2 is non-zero, else 0
 *       (only the WPO weights use it, and it costs the kernel one more multiply-add per logit)
 *   [2] 1 if index[r, 0] is the row's arg-max (the FIRST maximal position, as torch.argmax), else 0
 *   [3] 0 (reserved)  An index outside [0, vocab) yields NaN for that entry and sets
 * TRLK_FLAG_INDEX_OUT_OF_RANGE in *d_error_flag.
 */
int trlk_logp_entropy_fwd(const void* d_logits, int dtype, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                          int64_t seq_stride, int64_t row_stride, const int64_t* d_index, int32_t n_index,
                          float temperature, const uint8_t* d_row_mask, float* d_out_logp, float* d_out_entropy,
                          float* d_out_lse, float* d_out_row_stats, int32_t row_stats_sum_p2, int32_t* d_error_flag,
                          trlk_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * K3  backward of K1 by recomputation from the saved lse: one read and one write of the
 * logits-sized data.  Replaces autograd's log_softmax / gather / div / slice backward chain
 * behind utils.py:506-518 and grpo_trainer.py:1514-1519:
 *   dlogits[r, v] = ( sum_k g_logp[r,k] * (1[v == index[r,k]] - p_v)
 *                     - g_entropy[r] * p_v * ((z_v - lse_r) + H_r) ) / temperature,  p_v = exp(z_v - lse_r)
 * The output is a strided [n_seq, out_rows_per_seq, vocab] tensor of the same dtype as the
 * logits; the rows_per_seq input rows of a sequence land at output rows
 * [out_row_offset, out_row_offset + rows_per_seq) and every other output row is zero-filled
 * (the zero padding of the slice backward).  Rows whose upstream gradients are all exactly
 * zero are zero-filled without reading the logits.
 * d_g_entropy and d_entropy may be NULL together (no entropy gradient).
 */
int trlk_logp_entropy_bwd(const void* d_logits, int dtype, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                          int64_t seq_stride, int64_t row_stride, const int64_t* d_index, int32_t n_index,
                          float temperature, const float* d_lse, const float* d_entropy, const float* d_g_logp,
                          const float* d_g_entropy, void* d_dlogits, int64_t out_rows_per_seq, int64_t out_row_offset,
                          int64_t out_seq_stride, int64_t out_row_stride, trlk_stream_t stream);

/* fp64 logits (the float64 case of selective_log_softmax / entropy_from_logits, trl/trainer/utils.py:506-510,526-560,
 * which the reference's own unit tests run: tests/test_utils.py:866-905): the same two operations with double
 * operands, double arithmetic and double outputs.  Same argument meaning as the entry points above; no row
 * statistics.  Written for exactness (two sweeps per row), not for bandwidth. */
int trlk_logp_entropy_fwd_f64(const double* d_logits, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                              int64_t seq_stride, int64_t row_stride, const int64_t* d_index, int32_t n_index,
                              double temperature, const uint8_t* d_row_mask, double* d_out_logp, double* d_out_entropy,
                              double* d_out_lse, int32_t* d_error_flag, trlk_stream_t stream);
int trlk_logp_entropy_bwd_f64(const double* d_logits, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                              int64_t seq_stride, int64_t row_stride, const int64_t* d_index, int32_t n_index,
                              double temperature, const double* d_lse, const double* d_entropy, const double* d_g_logp,
                              const double* d_g_entropy, double* d_dlogits, int64_t out_rows_per_seq,
                              int64_t out_row_offset, int64_t out_seq_stride, int64_t out_row_stride,
                              trlk_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * K2a  group-relative advantages (trl/trainer/grpo_trainer.py:2685-2707, 2730 with nanstd,
 * trl/trainer/utils.py:874-880).  d_rewards fp32 [n] (NaN = unscorable), groups are
 * `group_size` consecutive entries, n % group_size == 0.
 *   adv = (r - nanmean_group) / (nanstd + 1e-4), NaN -> 0; nanstd per group, over the batch,
 *   or no division, per `scale_mode` (trlk_scale_rewards).
 */
int trlk_group_advantages(const float* d_rewards, int64_t n, int32_t group_size, int32_t scale_mode,
                          float* d_out_advantages, trlk_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * K2  GRPO clipped-surrogate loss, its metrics and d(loss)/d(logp) in one call
 * (trl/trainer/grpo_trainer.py:3054-3150, :3155-3181 entropy bonus, :3224-3258 metrics).
 * All [B, T] operands are dense fp32.  `loss_type` picks the normalisation (cispo and vespo use
 * TRLK_DAPO, sapo uses TRLK_GRPO), `policy_term` the per-token term, `sequence_level` != 0 the
 * sequence-level importance weight exp(masked mean of logp - old_logp) (:3057-3059).
 *   d_old_logp  NULL  -> old = logp (on-policy, :3037)
 *   d_ref_logp  NULL  -> requires beta == 0
 *   d_entropy   NULL  -> no entropy metric / bonus
 *   d_token_weight NULL -> 1; otherwise multiplies the policy term before the KL is added
 *                  (product of the off-policy, entropy-quantile and importance-sampling
 *                  factors of :3111-3118)
 *   d_entropy_mask NULL -> 1; extra factor on the mask of the entropy bonus (:3158)
 *   d_seq_coef  fp32 [B], only for TRLK_TERM_WEIGHTED_LOGP
 *   advantages: element (b, t) at d_advantages[b*adv_stride_b + t*adv_stride_t]
 *   delta: NaN = no upper clamp of the ratio (:3086-3087)
 *   d_dapo_normalizer: device scalar holding num_items_in_batch (DAPO only, :3140)
 *   dr_grpo_denominator: B * max_completion_length (:3135)
 * Outputs: d_out_loss [1]; d_out_metrics [TRLK_GRPO_NUM_METRICS]; d_out_dlogp [B, T] =
 * d loss / d logp; d_out_dentropy [B, T] (may be NULL unless entropy_coef != 0).
 * Reductions run in a fixed order: results are bit-reproducible.
 * d_workspace: trlk_grpo_workspace_bytes(B) bytes.
 */
enum trlk_grpo_metric {
    TRLK_M_KL_MEAN = 0,          /* masked mean of the k3 KL (NaN if beta == 0) */
    TRLK_M_ENTROPY_MEAN = 1,     /* masked mean entropy (NaN if no entropy given) */
    TRLK_M_CLIP_LOW_MEAN = 2,
    TRLK_M_CLIP_HIGH_MEAN = 3,
    TRLK_M_CLIP_REGION_MEAN = 4,
    TRLK_M_CLIP_LOW_MIN = 5,     /* min over sequences of the per-sequence mean, NaN rows skipped */
    TRLK_M_CLIP_HIGH_MAX = 6,
    TRLK_M_POLICY_LOSS = 7,      /* loss before the entropy bonus and before /grad_accum (:3127) */
    TRLK_M_MASK_SUM = 8,
    TRLK_M_KL_SUM = 9,
    TRLK_M_ENTROPY_SUM = 10,
    TRLK_M_AUX_MEAN = 11,        /* cispo: clip ratio (:3255-3256); weighted-logp: mean coefficient (:3258) */
    TRLK_M_CLIP_COUNT = 12,      /* denominator of the clip means: mask sum, or B with sequence-level weights */
    TRLK_M_AUX_SUM = 13,
    TRLK_M_AUX_COUNT = 14,
    TRLK_GRPO_NUM_METRICS = 16
};

size_t trlk_grpo_workspace_bytes(int64_t n_seq);

int trlk_grpo_loss(const float* d_logp, const float* d_old_logp, const float* d_ref_logp, const float* d_entropy,
                   const float* d_advantages, int64_t adv_stride_b, int64_t adv_stride_t, const float* d_mask,
                   const float* d_token_weight, const float* d_entropy_mask, const float* d_seq_coef, int64_t n_seq,
                   int64_t seq_len, int32_t loss_type, int32_t policy_term, int32_t sequence_level, float epsilon_low,
                   float epsilon_high, float delta, float beta, int32_t use_bias_correction_kl, float grad_accum_steps,
                   float dr_grpo_denominator, const float* d_dapo_normalizer, float num_processes, float entropy_coef,
                   float sapo_temperature_pos, float sapo_temperature_neg, float* d_out_loss, float* d_out_metrics,
                   float* d_out_dlogp, float* d_out_dentropy, void* d_workspace, size_t workspace_bytes,
                   trlk_stream_t stream);

/* trlk_grpo_loss_static: trlk_grpo_loss without the workspace argument, for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The per-sequence partial sums live in a device array built into the library
 * (512 KiB per GPU, held until the process ends), so n_seq is limited to trlk_grpo_loss_static_max_seq() = 8192;
 * more sequences are rejected with TRLK_ERR_WORKSPACE.  The call allocates and frees nothing.  All calls on one GPU
 * share that GPU's array: calls that overlap on one GPU (different streams or threads) race and must be serialised by
 * the caller.  Same arguments, outputs and bit-exact results as trlk_grpo_loss.
 * trlk_init looks up the array's address on the current device (once per device); a caller that captures graphs
 * calls it beforehand, with each device current -- otherwise the first trlk_grpo_loss_static call on a device does it.
 * trlk_init also allows the builds of trlk_grpo_fused_fwd_bwd that keep part of a row in LDS (rows above 163840
 * 16-bit or 81920 fp32 logits) their LDS on the current device, which otherwise happens at the first such launch. */
int trlk_init(void);
int64_t trlk_grpo_loss_static_max_seq(void);
int trlk_grpo_loss_static(const float* d_logp, const float* d_old_logp, const float* d_ref_logp, const float* d_entropy,
                          const float* d_advantages, int64_t adv_stride_b, int64_t adv_stride_t, const float* d_mask,
                          const float* d_token_weight, const float* d_entropy_mask, const float* d_seq_coef,
                          int64_t n_seq, int64_t seq_len, int32_t loss_type, int32_t policy_term, int32_t sequence_level,
                          float epsilon_low, float epsilon_high, float delta, float beta, int32_t use_bias_correction_kl,
                          float grad_accum_steps, float dr_grpo_denominator, const float* d_dapo_normalizer,
                          float num_processes, float entropy_coef, float sapo_temperature_pos,
                          float sapo_temperature_neg, float* d_out_loss, float* d_out_metrics, float* d_out_dlogp,
                          float* d_out_dentropy, trlk_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * K4  sequence-level losses on top of per-token log-probs.
 *
 * trlk_dpo_loss: DPO sequence log-probs and sigmoid loss (trl/trainer/dpo_trainer.py:1348-1350,
 * 1362, 1396-1402, 1430-1435, 1578).  d_token_logp, d_mask: dense fp32 [n_seq, seq_len]
 * (already shifted); n_seq is even, first half chosen, second half rejected.
 *   seq[b]  = sum_t logp[b,t] * 1[mask[b,t] != 0]
 *   delta_p = (seq_c - ref_c) - (seq_r - ref_r);  loss = mean_p -logsigmoid(beta * delta_p)
 * Outputs: d_out_seq_logps [n_seq], d_out_loss [1], d_out_metrics [TRLK_DPO_NUM_METRICS],
 * d_out_dlogp [n_seq, seq_len] = d loss / d token_logp.
 */
enum trlk_dpo_metric {
    TRLK_D_REWARD_CHOSEN = 0,    /* mean beta*(seq_c - ref_c)   (dpo_trainer.py:1634-1639) */
    TRLK_D_REWARD_REJECTED = 1,
    TRLK_D_REWARD_ACCURACY = 2,
    TRLK_D_REWARD_MARGIN = 3,
    TRLK_D_LOGPS_CHOSEN = 4,
    TRLK_D_LOGPS_REJECTED = 5,
    TRLK_DPO_NUM_METRICS = 8
};

int trlk_dpo_loss(const float* d_token_logp, const float* d_mask, const float* d_ref_chosen,
                  const float* d_ref_rejected, int64_t n_seq, int64_t seq_len, float beta, float* d_out_seq_logps,
                  float* d_out_loss, float* d_out_metrics, float* d_out_dlogp, trlk_stream_t stream);

/* trlk_rloo_loss: RLOO sequence-level clipped loss (trl/trainer/rloo_trainer.py:1683-1694,
 * 1711-1721).  seq[b] = sum_t logp*mask; ratio = exp(seq - old_seq); loss = mean_b
 * -min(ratio*A, clamp(ratio, 1-eps_low, 1+eps_high)*A).
 * Metrics: [0] low_mean [1] low_min [2] high_mean [3] high_max [4] region_mean.
 */
#define TRLK_RLOO_NUM_METRICS 8
int trlk_rloo_loss(const float* d_token_logp, const float* d_mask, const float* d_old_seq_logps,
                   const float* d_advantages, int64_t n_seq, int64_t seq_len, float epsilon_low, float epsilon_high,
                   float* d_out_seq_logps, float* d_out_loss, float* d_out_metrics, float* d_out_dlogp,
                   trlk_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * K5 / K6  lm_head fused with the log-prob / entropy reduction; the [N, V] logits are never
 * written to memory.  Replaces _ChunkedLogProbFunction (trl/trainer/utils.py:1291-1424):
 *   y = hidden @ weight^T (+ bias)  (bf16/fp16 operands on the matrix cores, fp32 accumulation;
 *       d_bias: optional fp32 [vocab], the lm_head bias the fused-linear operators behind
 *       use_liger_kernel take, trl/trainer/grpo_trainer.py:2885-2896, dpo_trainer.py:1287-1289)
 *   z = softcap(y * logit_scale) / temperature,  softcap(x) = cap * tanh(x / cap) if cap > 0
 *   out_logp[n] = z[n, targets[n]] - logsumexp(z[n, :]);  out_entropy[n] = logsumexp - E_p[z];
 *   out_log_z[n] = logsumexp(z[n, :])   (saved for the backward)
 * d_hidden [n_tokens, hidden_size] and d_weight [vocab, hidden_size] are row-major with row
 * strides (elements) that are multiples of 8, 16-byte aligned; dtype TRLK_BF16 or TRLK_F16.
 * Unlike the reference, the logits are not rounded to the operand dtype before the reduction.
 * A target outside [0, vocab) yields NaN and sets TRLK_FLAG_INDEX_OUT_OF_RANGE.
 * d_out_target_is_max (optional, fp32 [n_tokens]): 1 where the target's logit is the row maximum, i.e.
 * argmax(logits) == target up to ties -- the token-accuracy count of the chunked cross-entropy
 * (trl/trainer/sft_trainer.py:99-114) comes out of the same pass.
 */
size_t trlk_fused_head_fwd_workspace_bytes(int64_t n_tokens);

/* Optional stash of the forward's softmax numerators: for every logit exp(z - reference) as fp16, where the
 * reference is the running maximum the forward held when it summed that part of the row (kept beside the
 * numerators, one fp32 per 64 logits), plus the target's logit of every token.  The layout is the library's own
 * (vocabulary-major, rows of *out_ld tokens, *out_ld = n_tokens rounded up to 256; `stash_ld` below is that number).
 * A forward that is given the buffer (d_out_stash, stash_ld) fills it; a backward that is given the same buffer
 * (d_stash), `vocab` and the other arguments of that forward derives dz from it in one memory-bound sweep (one
 * multiplication per logit) instead of recomputing the chunk's logits on the matrix cores (a third of the backward's
 * work).  fp16 keeps 11 significant bits of every probability down to 2^-29 of the row's running maximum and nothing
 * below 2^-39 of it: what dz keeps anyway once it is rounded to fp16 for the two products.  No counterpart in the
 * reference, which always recomputes (trl/trainer/utils.py:1385-1399): it trades about vocab * n_tokens * 2.07 bytes
 * held between forward and backward for that recompute.  Returns the buffer size in bytes; the buffer must be
 * 16-byte aligned.
 */
size_t trlk_fused_head_stash_bytes(int64_t n_tokens, int64_t vocab, int64_t* out_ld);

int trlk_fused_head_fwd(const void* d_hidden, const void* d_weight, const int64_t* d_targets, int dtype,
                        int64_t n_tokens, int64_t vocab, int64_t hidden_size, int64_t hidden_stride,
                        int64_t weight_stride, float temperature, float final_logit_softcapping, float logit_scale,
                        const float* d_bias, float* d_out_logp, float* d_out_entropy, float* d_out_log_z,
                        float* d_out_target_is_max, void* d_out_stash, int64_t stash_ld, int32_t* d_error_flag,
                        void* d_workspace, size_t workspace_bytes, trlk_stream_t stream);

/* Backward of the above w.r.t. hidden and weight for an upstream gradient on the log-probs
 * (the entropy output carries no gradient, as in the reference, utils.py:1368):
 *   dz[n, v] = g[n] * (1[v == targets[n]] - exp(z[n, v] - log_z[n])) * d z / d y
 *   out_dhidden = dz @ weight,  out_dweight = dz^T @ hidden   (fp32 accumulation, outputs in `dtype`,
 *   dense [n_tokens, hidden_size] and [vocab, hidden_size]).
 * The vocabulary is processed in chunks of `chunk_size` rows (rounded up to 256); dz exists only
 * for one chunk at a time inside the workspace, as fp16 whatever `dtype` is: both products run on
 * fp16 operands (11 significant bits in dz instead of bf16's 8; the reference keeps fp32 grad_logits,
 * utils.py:1405-1424), each operand multiplied by a power of two taken from its largest magnitude
 * (dz per token, hidden^T's columns by the inverse of that relative to the largest |g|, and for bf16 inputs
 * W_chunk^T and hidden^T by their own maxima, which convert exactly) and the factors divided out of the fp32
 * accumulators, so that neither small upstream gradients nor wide-ranged bf16 values leave the fp16 range.
 * d_out_dbias (optional, fp32 [vocab]): sum over tokens of dz, the gradient of d_bias.
 * d_stash_cols (optional, int32 [n_tokens]): the stash column of each token, for a caller that dropped tokens
 * since the forward (those without an upstream gradient contribute nothing to either product); values in
 * [0, stash_ld).
 */
size_t trlk_fused_head_bwd_workspace_bytes(int64_t n_tokens, int64_t vocab, int64_t hidden_size, int64_t chunk_size);

int trlk_fused_head_bwd(const void* d_hidden, const void* d_weight, const int64_t* d_targets, int dtype,
                        int64_t n_tokens, int64_t vocab, int64_t hidden_size, int64_t hidden_stride,
                        int64_t weight_stride, float temperature, float final_logit_softcapping, float logit_scale,
                        const float* d_bias, const float* d_log_z, const float* d_g_logp, int64_t chunk_size,
                        const void* d_stash, int64_t stash_ld, const int32_t* d_stash_cols, void* d_out_dhidden,
                        void* d_out_dweight, float* d_out_dbias, void* d_workspace, size_t workspace_bytes,
                        trlk_stream_t stream);

/* fp32 operands of the fused head (the dtype of the reference's own unit test of _ChunkedLogProbFunction,
 * tests/test_utils.py:1161-1232; the reference runs `torch.mm(last_hidden, w_chunk.t())` in the operands'
 * dtype and the two backward products in fp32, trl/trainer/utils.py:1327-1328,1421-1422).  The matrix cores take 16-bit operands, so an
 * fp32 matrix is split into three bf16 pieces (24 significant bits in all, fp32's exponent range) laid out along
 * the contraction axis: trlk_split_bf16x3 turns fp32 [rows, cols] into bf16 [rows, 6 * cpad] (cpad = cols rounded
 * up to 8, padding zero-filled; side 0 for the left operand of an NT product, 1 for the right one), and an NT
 * product of a side-0 and a side-1 matrix over the 6 * cpad columns is the fp32 product to fp32 rounding.  The
 * forward runs trlk_fused_head_fwd on such pieces (hidden_size = 6 * cpad); trlk_gemm_nt is the plain product
 * C[m, n] (+)= A[m, k] * B[n, k]^T (16-bit operands with k contiguous, fp32 output) for the backward's logits
 * recompute and its two gradient products on pieces of d logits.
 */
int trlk_split_bf16x3(const float* d_in, int64_t rows, int64_t cols, int64_t ld_in, int side, void* d_out,
                      int64_t ld_out, trlk_stream_t stream);
int trlk_gemm_nt(const void* d_a, int64_t lda, const void* d_b, int64_t ldb, int dtype, int64_t m, int64_t n,
                 int64_t k, float* d_out, int64_t ldo, int accumulate, trlk_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * K7  GRPO loss gradient straight from the logits: one read and one write of the logits-sized
 * data instead of K1 + K3's two reads and one write.  Stands in for the whole chain
 * `_get_per_token_logps_and_entropies` -> `_compute_loss` -> `loss.backward()` down to dlogits
 * (trl/trainer/grpo_trainer.py:1514-1532, 3026-3150) for the token-level loss types, where the
 * gradient coefficient of a token depends only on its own log-prob, on per-token inputs and on
 * normalisers known from the mask:
 *   d_row_scale fp32 [n_seq] = d loss / d (masked token loss of that sequence), e.g. 1 / num_items for dapo;
 *   d_entropy_weight fp32 [n_seq, rows_per_seq] or NULL = d loss / d entropy of each token (the entropy bonus of
 *   grpo_trainer.py:3155-3181 with its normaliser folded in);
 *   the other per-token inputs, the policy terms and their parameters are those of trlk_grpo_loss.
 * bf16, fp16 or fp32 logits, vocab <= trlk_grpo_fused_max_vocab(dtype) (a row is held
 * in the registers of one workgroup, the end of a row of more than 163840 logits in its LDS, and what
 * lies beyond 237568 logits is read twice); rows that are not whole aligned 16-byte vectors are peeled to
 * their alignment (at least two vectors' worth of entries then).  Outputs: log-prob, entropy and lse of
 * every row of the completion mask (the others are not read and yield 0, unless compute_masked_rows
 * asks for their outputs too), and the full
 * [n_seq, out_rows_per_seq, vocab] gradient laid out as trlk_logp_entropy_bwd writes it, for an
 * upstream gradient of 1 on the loss.  trlk_scale_unless_one multiplies such a buffer by a device
 * scalar, and launches an empty kernel when that scalar is exactly 1.
 */
int64_t trlk_grpo_fused_max_vocab(int dtype);
int trlk_grpo_fused_fwd_bwd(const void* d_logits, int dtype, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                            int64_t seq_stride, int64_t row_stride, const int64_t* d_index, float temperature,
                            const float* d_old_logp, const float* d_ref_logp, const float* d_advantages,
                            int64_t adv_stride_b, int64_t adv_stride_t, const float* d_mask,
                            const float* d_token_weight, const float* d_seq_coef, const float* d_row_scale,
                            const float* d_entropy_weight, int policy_term, float epsilon_low, float epsilon_high, float delta, float beta,
                            int use_bias_correction_kl, float sapo_temperature_pos, float sapo_temperature_neg,
                            float* d_out_logp, float* d_out_entropy, float* d_out_lse, void* d_dlogits,
                            int64_t out_rows_per_seq, int64_t out_row_offset, int64_t out_seq_stride,
                            int64_t out_row_stride, int compute_masked_rows, int32_t* d_error_flag,
                            trlk_stream_t stream);
int trlk_scale_unless_one(void* d_data, int dtype, int64_t n_elems, const float* d_scale, trlk_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TRLK_H */

// K2 / K2a / K4: the [B, T]-sized loss epilogues (GRPO clipped surrogate + k3 KL + metrics,
// group-relative advantages, DPO sigmoid loss, RLOO sequence loss) and their gradients
// w.r.t. the per-token log-probs.  These touch ~40 bytes per token, nothing next to the
// vocabulary-sized passes, so the design goal is determinism and launch count, not bandwidth:
// every reduction has a fixed combination order (no float atomics), one workgroup owns one
// sequence, and the final cross-sequence reduction is recomputed identically by every
// workgroup instead of being passed through a third launch.
#include <mutex>

#include "common.hpp"
#include "grpo_token.hpp"

namespace trlk {
namespace {

constexpr int kThreads = 256;
constexpr int kRowStats = 16;  // floats of workspace per sequence

enum RowStat { RS_MASK = 0, RS_LOSS, RS_KL, RS_ENT, RS_LOW, RS_HIGH, RS_REGION, RS_ENT_EFF, RS_EFF, RS_QUOT };

// ------------------------------------------------------------------------------ advantages
__global__ __launch_bounds__(kThreads) void group_advantages_kernel(const float* __restrict__ rewards, int64_t n,
                                                                    int G, int mode, float* __restrict__ adv) {
    __shared__ float scratch[kThreads / kWave];
    const int tid = threadIdx.x;
    float batch_std = 0.f;
    if (mode == TRLK_SCALE_BATCH) {
        // nanstd over the whole batch: mean of the non-NaN entries, then Bessel-corrected variance
        float s = 0.f, cnt = 0.f;
        for (int64_t i = tid; i < n; i += kThreads) {
            const float r = rewards[i];
            if (r == r) {
                s += r;
                cnt += 1.f;
            }
        }
        s = block_sum<kThreads>(s, scratch);
        cnt = block_sum<kThreads>(cnt, scratch);
        const float mean = s / cnt;
        float q = 0.f;
        for (int64_t i = tid; i < n; i += kThreads) {
            const float r = rewards[i];
            if (r == r) q += (r - mean) * (r - mean);
        }
        q = block_sum<kThreads>(q, scratch);
        batch_std = (n > 1) ? ((cnt > 1.f) ? sqrtf(q / cnt * (cnt / (cnt - 1.f))) : NAN) : 0.f;
    }
    const int64_t n_groups = n / G;
    for (int64_t g = tid; g < n_groups; g += kThreads) {
        const float* r = rewards + g * G;
        float s = 0.f, cnt = 0.f;
        for (int i = 0; i < G; ++i)
            if (r[i] == r[i]) {
                s += r[i];
                cnt += 1.f;
            }
        const float mean = s / cnt;  // 0/0 = NaN for a group with no scorable entry
        float std_g = 0.f;
        if (mode == TRLK_SCALE_GROUP && G > 1) {
            float q = 0.f;
            for (int i = 0; i < G; ++i)
                if (r[i] == r[i]) q += (r[i] - mean) * (r[i] - mean);
            std_g = (cnt > 1.f) ? sqrtf(q / cnt * (cnt / (cnt - 1.f))) : NAN;
        }
        for (int i = 0; i < G; ++i) {
            float a = r[i] - mean;
            if (mode == TRLK_SCALE_GROUP) a = a / (std_g + 1e-4f);
            if (mode == TRLK_SCALE_BATCH) a = a / (batch_std + 1e-4f);
            adv[g * G + i] = (a == a) ? a : 0.f;
        }
    }
}

// ------------------------------------------------------------------------------ GRPO
struct GrpoArgs {
    const float *logp, *old_logp, *ref_logp, *entropy, *adv, *mask, *token_weight, *entropy_mask, *seq_coef;
    int64_t adv_stride_b, adv_stride_t;
    int64_t B, T;
    int loss_type, policy_term, seq_level;
    int luspo_dense;  // LUSPO whose per-token term is [B, T]: every position counts, the padding too (:3143-3148)
    float eps_low, eps_high, delta, beta;
    int bias_kl;
    float grad_accum, dr_denominator;
    const float* dapo_normalizer;
    float num_processes, entropy_coef, sapo_tau_pos, sapo_tau_neg;
    float *out_loss, *out_metrics, *out_dlogp, *out_dentropy, *ws;
};

constexpr int kRowStatsUsed = 13;
enum RowStat2 { RS_CLIP_CNT = 10, RS_AUX = 11, RS_AUX_CNT = 12 };
static_assert(kRowStatsUsed <= 16, "row stats");

// Pass 1: one workgroup per sequence.  Writes d(per-token loss)/d(logp) * mask (not yet
// normalised) and the sequence's masked sums.
__global__ __launch_bounds__(kThreads) void grpo_rows_kernel(GrpoArgs a) {
    __shared__ float scratch[kThreads / kWave];
    const int64_t b = blockIdx.x;
    const int tid = threadIdx.x;
    const int64_t off = b * a.T;
    const float coef = a.seq_coef ? a.seq_coef[b] : 0.f;

    // sequence-level importance weight: exp(masked mean of the token log-ratios)   (:3057-3059)
    float n_b = 0.f, c_seq = 1.f;
    if (a.seq_level || a.luspo_dense) {
        float s1 = 0.f, s0 = 0.f;
        for (int64_t t = tid; t < a.T; t += kThreads) {
            const float m = a.mask[off + t];
            if (m == 0.f) continue;
            s0 += m;
            if (a.seq_level && a.old_logp) s1 += (a.logp[off + t] - a.old_logp[off + t]) * m;
        }
        s1 = block_sum<kThreads>(s1, scratch);
        n_b = block_sum<kThreads>(s0, scratch);
        c_seq = expf(s1 / fmaxf(n_b, 1.f));
    }
    // with per-token advantages the clip flags of a sequence-level ratio are per token again (:3237-3250)
    const bool seq_flags = a.seq_level && a.adv_stride_t == 0;

    float s_mask = 0, s_loss = 0, s_kl = 0, s_ent = 0, s_low = 0, s_high = 0, s_reg = 0, s_ent_eff = 0, s_eff = 0;
    float s_aux = 0, s_glnc = 0;
    for (int64_t t = tid; t < a.T; t += kThreads) {
        const float m = a.mask[off + t];
        // weight of the token in the loss: the mask, except for the [B, T] form of LUSPO, which averages over
        // every position of the padded batch
        const float ml = a.luspo_dense ? 1.f : m;
        if (ml == 0.f) {  // a masked token contributes exactly nothing, whatever its (possibly skipped) inputs hold
            a.out_dlogp[off + t] = 0.f;
            continue;
        }
        const float lp = a.logp[off + t];
        const float A = a.adv[b * a.adv_stride_b + t * a.adv_stride_t];
        const float c_raw = a.seq_level ? c_seq : (a.old_logp ? expf(lp - a.old_logp[off + t]) : 1.f);
        const PolicyTerm p = policy_term(a, c_raw, A, lp, coef);
        float pl, kl, g_lnc, g_lp;
        grpo_token_terms(a, p, c_raw, lp, a.token_weight ? a.token_weight[off + t] : 1.f,
                         a.beta != 0.f ? a.ref_logp[off + t] : 0.f, pl, kl, g_lnc, g_lp);
        const float H = a.entropy ? a.entropy[off + t] : 0.f;
        const float eff = a.entropy_mask ? m * a.entropy_mask[off + t] : m;
        s_mask += m;
        s_loss += pl * ml;
        s_kl += kl * m;
        s_ent += H * m;
        s_low += p.low * m;
        s_high += p.high * m;
        s_reg += fmaxf(p.low, p.high) * m;
        s_aux += p.aux * m;
        s_ent_eff += H * eff;
        s_eff += eff;
        if (a.seq_level) {
            s_glnc += g_lnc * ml;
            a.out_dlogp[off + t] = g_lp * ml;
        } else {
            a.out_dlogp[off + t] = (g_lp + g_lnc) * ml;
        }
    }
    float* ws = a.ws + b * kRowStats;
    const float r_mask = block_sum<kThreads>(s_mask, scratch);
    float r_loss = block_sum<kThreads>(s_loss, scratch);
    if (a.luspo_dense) r_loss *= r_mask;  // every position's term times the sequence's active-token count
    const float r_kl = block_sum<kThreads>(s_kl, scratch);
    const float r_ent = block_sum<kThreads>(s_ent, scratch);
    float r_low = block_sum<kThreads>(s_low, scratch);
    float r_high = block_sum<kThreads>(s_high, scratch);
    float r_reg = block_sum<kThreads>(s_reg, scratch);
    float r_aux = block_sum<kThreads>(s_aux, scratch);
    const float r_ent_eff = block_sum<kThreads>(s_ent_eff, scratch);
    const float r_eff = block_sum<kThreads>(s_eff, scratch);
    float clip_cnt = r_mask, aux_cnt = r_mask;
    if (a.seq_level) {
        // the ratio-dependent part of every token's loss pulls on all tokens of the sequence through the mean
        const float g_seq = block_sum<kThreads>(s_glnc, scratch) / fmaxf(n_b, 1.f);
        for (int64_t t = tid; t < a.T; t += kThreads) {
            const float m = a.mask[off + t];
            if (m != 0.f) a.out_dlogp[off + t] += g_seq * m;
        }
    }
    if (seq_flags) {
        // clip flags are per sequence: one value each, also for a sequence without active tokens
        const PolicyTerm p = policy_term(a, c_seq, a.adv[b * a.adv_stride_b], 0.f, coef);
        r_low = p.low;
        r_high = p.high;
        r_reg = fmaxf(p.low, p.high);
        r_aux = p.aux;
        clip_cnt = 1.f;
        aux_cnt = 1.f;
    }
    if (a.policy_term == TRLK_TERM_WEIGHTED_LOGP) {  // the logged quantity is the per-sequence coefficient
        r_aux = coef;
        aux_cnt = 1.f;
    }
    if (tid == 0) {
        ws[RS_MASK] = r_mask;
        ws[RS_LOSS] = r_loss;
        ws[RS_KL] = r_kl;
        ws[RS_ENT] = r_ent;
        ws[RS_LOW] = r_low;
        ws[RS_HIGH] = r_high;
        ws[RS_REGION] = r_reg;
        ws[RS_ENT_EFF] = r_ent_eff;
        ws[RS_EFF] = r_eff;
        ws[RS_QUOT] = r_loss / fmaxf(r_mask, 1.f);
        ws[RS_CLIP_CNT] = clip_cnt;
        ws[RS_AUX] = r_aux;
        ws[RS_AUX_CNT] = aux_cnt;
    }
}

// Pass 2: every workgroup re-reduces the per-sequence sums in the same order (so all of them
// hold bit-identical totals), workgroup 0 writes loss and metrics, and each workgroup
// normalises the gradient row of its own sequence.
__global__ __launch_bounds__(kThreads) void grpo_finish_kernel(GrpoArgs a) {
    __shared__ float scratch[kThreads / kWave];
    const int64_t b = blockIdx.x;
    const int tid = threadIdx.x;
    float tot[kRowStatsUsed];
#pragma unroll
    for (int j = 0; j < kRowStatsUsed; ++j) tot[j] = 0.f;
    float low_min = INFINITY, high_max = -INFINITY;
    for (int64_t r = tid; r < a.B; r += kThreads) {
        const float* ws = a.ws + r * kRowStats;
#pragma unroll
        for (int j = 0; j < kRowStatsUsed; ++j) tot[j] += ws[j];
        const float lm = ws[RS_LOW] / ws[RS_CLIP_CNT], hm = ws[RS_HIGH] / ws[RS_CLIP_CNT];  // NaN for an empty sequence
        if (lm == lm) low_min = fminf(low_min, lm);
        if (hm == hm) high_max = fmaxf(high_max, hm);
    }
#pragma unroll
    for (int j = 0; j < kRowStatsUsed; ++j) tot[j] = block_sum<kThreads>(tot[j], scratch);
    low_min = wave_min(low_min);
    high_max = wave_max(high_max);
    __shared__ float s_min[kThreads / kWave], s_max[kThreads / kWave];
    if ((tid & (kWave - 1)) == 0) {
        s_min[tid / kWave] = low_min;
        s_max[tid / kWave] = high_max;
    }
    __syncthreads();
    for (int w = 0; w < kThreads / kWave; ++w) {
        low_min = fminf(low_min, s_min[w]);
        high_max = fmaxf(high_max, s_max[w]);
    }

    const float Bf = float(a.B);
    float norm_rows;  // d loss / d (sum of masked per-token losses), before the per-row factor
    float loss;
    const float dapo_norm = (a.loss_type == TRLK_DAPO) ? fmaxf(a.dapo_normalizer[0], 1.f) / a.num_processes : 1.f;
    switch (a.loss_type) {
        case TRLK_GRPO:
            loss = tot[RS_QUOT] / Bf;
            norm_rows = 1.f / Bf;  // times 1 / max(mask_sum_b, 1) per row
            break;
        case TRLK_LUSPO:  // mean over sequences of (per-sequence loss * active tokens)   (:3143-3148)
            loss = tot[RS_LOSS] / Bf;
            norm_rows = 1.f / Bf;
            if (a.luspo_dense) {  // the same mean taken over all B * T entries of a [B, T] term
                loss /= float(a.T);
                norm_rows /= float(a.T);
            }
            break;
        case TRLK_BNPO:
            loss = tot[RS_LOSS] / fmaxf(tot[RS_MASK], 1.f);
            norm_rows = 1.f / fmaxf(tot[RS_MASK], 1.f);
            break;
        case TRLK_DR_GRPO:
            loss = tot[RS_LOSS] / a.dr_denominator;
            norm_rows = 1.f / a.dr_denominator;
            break;
        default:  // TRLK_DAPO
            loss = tot[RS_LOSS] / dapo_norm;
            norm_rows = 1.f / dapo_norm;
            break;
    }
    const float policy_loss = loss;
    const float ga = (a.loss_type == TRLK_DAPO) ? 1.f : a.grad_accum;
    loss = loss / ga;
    norm_rows = norm_rows / ga;
    float ent_scale = 0.f;  // d loss / d entropy[b, t] = ent_scale * eff[b, t]
    if (a.entropy_coef != 0.f) {
        float term;
        if (a.loss_type == TRLK_DAPO) {
            term = tot[RS_ENT_EFF] / dapo_norm;
            ent_scale = -a.entropy_coef / dapo_norm;
        } else {
            term = tot[RS_ENT_EFF] / fmaxf(tot[RS_EFF], 1.f) / ga;
            ent_scale = -a.entropy_coef / fmaxf(tot[RS_EFF], 1.f) / ga;
        }
        loss -= a.entropy_coef * term;
    }
    if (b == 0 && tid == 0) {
        const float cnt = fmaxf(tot[RS_MASK], 1.f);
        const float clip_cnt = fmaxf(tot[RS_CLIP_CNT], 1.f);
        a.out_loss[0] = loss;
        float* mt = a.out_metrics;
        for (int j = 0; j < TRLK_GRPO_NUM_METRICS; ++j) mt[j] = 0.f;
        mt[TRLK_M_KL_MEAN] = (a.beta != 0.f) ? tot[RS_KL] / cnt : NAN;
        mt[TRLK_M_ENTROPY_MEAN] = a.entropy ? tot[RS_ENT] / cnt : NAN;
        mt[TRLK_M_CLIP_LOW_MEAN] = tot[RS_LOW] / clip_cnt;
        mt[TRLK_M_CLIP_HIGH_MEAN] = tot[RS_HIGH] / clip_cnt;
        mt[TRLK_M_CLIP_REGION_MEAN] = tot[RS_REGION] / clip_cnt;
        mt[TRLK_M_CLIP_LOW_MIN] = (low_min == INFINITY) ? NAN : low_min;
        mt[TRLK_M_CLIP_HIGH_MAX] = (high_max == -INFINITY) ? NAN : high_max;
        mt[TRLK_M_POLICY_LOSS] = policy_loss;
        mt[TRLK_M_MASK_SUM] = tot[RS_MASK];
        mt[TRLK_M_KL_SUM] = tot[RS_KL];
        mt[TRLK_M_ENTROPY_SUM] = tot[RS_ENT];
        mt[TRLK_M_AUX_MEAN] = tot[RS_AUX] / fmaxf(tot[RS_AUX_CNT], 1.f);
        mt[TRLK_M_CLIP_COUNT] = tot[RS_CLIP_CNT];
        mt[TRLK_M_AUX_SUM] = tot[RS_AUX];
        mt[TRLK_M_AUX_COUNT] = tot[RS_AUX_CNT];
    }
    const float row_scale = (a.loss_type == TRLK_GRPO) ? norm_rows / fmaxf(a.ws[b * kRowStats + RS_MASK], 1.f)
                            : a.luspo_dense           ? norm_rows * a.ws[b * kRowStats + RS_MASK]
                                                      : norm_rows;
    const int64_t off = b * a.T;
    for (int64_t t = tid; t < a.T; t += kThreads) {
        a.out_dlogp[off + t] *= row_scale;
        if (a.out_dentropy) {
            const float m = a.mask[off + t];
            const float eff = a.entropy_mask ? m * a.entropy_mask[off + t] : m;
            a.out_dentropy[off + t] = ent_scale * eff;
        }
    }
}

// ------------------------------------------------------------------------------ DPO / RLOO
// seq[b] = sum_t logp * (INDICATOR ? 1[mask != 0] : mask)
template <bool INDICATOR>
__global__ __launch_bounds__(kThreads) void masked_row_sum_kernel(const float* __restrict__ logp,
                                                                  const float* __restrict__ mask, int64_t T,
                                                                  float* __restrict__ seq) {
    __shared__ float scratch[kThreads / kWave];
    const int64_t off = int64_t(blockIdx.x) * T;
    float s = 0.f;
    for (int64_t t = threadIdx.x; t < T; t += kThreads) {
        const float m = mask[off + t];
        if (INDICATOR) {
            if (m != 0.f) s += logp[off + t];
        } else {
            s += logp[off + t] * m;
        }
    }
    s = block_sum<kThreads>(s, scratch);
    if (threadIdx.x == 0) seq[blockIdx.x] = s;
}

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }
__device__ __forceinline__ float sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

__global__ __launch_bounds__(kThreads) void dpo_finish_kernel(const float* __restrict__ seq,
                                                              const float* __restrict__ ref_c,
                                                              const float* __restrict__ ref_r,
                                                              const float* __restrict__ mask, int64_t B, int64_t T,
                                                              float beta, float* __restrict__ out_loss,
                                                              float* __restrict__ out_metrics,
                                                              float* __restrict__ out_dlogp) {
    __shared__ float scratch[kThreads / kWave];
    const int64_t P = B / 2;
    const int tid = threadIdx.x;
    const int64_t b = blockIdx.x;
    if (b == 0) {
        float s_loss = 0, s_rc = 0, s_rr = 0, s_acc = 0, s_lc = 0, s_lr = 0;
        for (int64_t p = tid; p < P; p += kThreads) {
            const float lc = seq[p] - ref_c[p], lr = seq[P + p] - ref_r[p];
            s_loss += -log_sigmoid(beta * (lc - lr));
            s_rc += beta * lc;
            s_rr += beta * lr;
            s_acc += (beta * lc > beta * lr) ? 1.f : 0.f;
            s_lc += seq[p];
            s_lr += seq[P + p];
        }
        s_loss = block_sum<kThreads>(s_loss, scratch);
        s_rc = block_sum<kThreads>(s_rc, scratch);
        s_rr = block_sum<kThreads>(s_rr, scratch);
        s_acc = block_sum<kThreads>(s_acc, scratch);
        s_lc = block_sum<kThreads>(s_lc, scratch);
        s_lr = block_sum<kThreads>(s_lr, scratch);
        if (tid == 0) {
            const float Pf = float(P);
            out_loss[0] = s_loss / Pf;
            for (int j = 0; j < TRLK_DPO_NUM_METRICS; ++j) out_metrics[j] = 0.f;
            out_metrics[TRLK_D_REWARD_CHOSEN] = s_rc / Pf;
            out_metrics[TRLK_D_REWARD_REJECTED] = s_rr / Pf;
            out_metrics[TRLK_D_REWARD_ACCURACY] = s_acc / Pf;
            out_metrics[TRLK_D_REWARD_MARGIN] = (s_rc - s_rr) / Pf;
            out_metrics[TRLK_D_LOGPS_CHOSEN] = s_lc / Pf;
            out_metrics[TRLK_D_LOGPS_REJECTED] = s_lr / Pf;
        }
    }
    // d loss / d seq: -beta * sigmoid(-beta * delta) / P for the chosen row, + for the rejected one
    const int64_t p = (b < P) ? b : b - P;
    const float delta = (seq[p] - ref_c[p]) - (seq[P + p] - ref_r[p]);
    const float g = beta * sigmoid(-beta * delta) / float(P) * ((b < P) ? -1.f : 1.f);
    const int64_t off = b * T;
    for (int64_t t = tid; t < T; t += kThreads) out_dlogp[off + t] = (mask[off + t] != 0.f) ? g : 0.f;
}

__global__ __launch_bounds__(kThreads) void rloo_finish_kernel(const float* __restrict__ seq,
                                                               const float* __restrict__ old_seq,
                                                               const float* __restrict__ adv,
                                                               const float* __restrict__ mask, int64_t B, int64_t T,
                                                               float eps_low, float eps_high,
                                                               float* __restrict__ out_loss,
                                                               float* __restrict__ out_metrics,
                                                               float* __restrict__ out_dlogp) {
    __shared__ float scratch[kThreads / kWave];
    const int tid = threadIdx.x;
    const int64_t b = blockIdx.x;
    const float lo = 1.f - eps_low, hi = 1.f + eps_high;
    if (b == 0) {
        float s_loss = 0, s_low = 0, s_high = 0, s_reg = 0;
        for (int64_t r = tid; r < B; r += kThreads) {
            const float c1 = expf(seq[r] - old_seq[r]);
            const float c2 = fminf(fmaxf(c1, lo), hi);
            const float A = adv[r];
            s_loss += -fminf(c1 * A, c2 * A);
            const float l = (c1 < lo && A < 0.f) ? 1.f : 0.f, h = (c1 > hi && A > 0.f) ? 1.f : 0.f;
            s_low += l;
            s_high += h;
            s_reg += fmaxf(l, h);
        }
        s_loss = block_sum<kThreads>(s_loss, scratch);
        s_low = block_sum<kThreads>(s_low, scratch);
        s_high = block_sum<kThreads>(s_high, scratch);
        s_reg = block_sum<kThreads>(s_reg, scratch);
        if (tid == 0) {
            const float Bf = float(B);
            out_loss[0] = s_loss / Bf;
            for (int j = 0; j < TRLK_RLOO_NUM_METRICS; ++j) out_metrics[j] = 0.f;
            out_metrics[0] = s_low / Bf;
            out_metrics[1] = (s_low == Bf) ? 1.f : 0.f;  // min of 0/1 flags (counts are exact in fp32)
            out_metrics[2] = s_high / Bf;
            out_metrics[3] = (s_high > 0.f) ? 1.f : 0.f;  // max of 0/1 flags
            out_metrics[4] = s_reg / Bf;
        }
    }
    const float c1 = expf(seq[b] - old_seq[b]);
    const float c2 = fminf(fmaxf(c1, lo), hi);
    const float A = adv[b];
    const float l1 = c1 * A, l2 = c2 * A;
    const float d1 = A * c1;
    const float d2 = (c1 >= lo && c1 <= hi) ? A * c1 : 0.f;
    const float w1 = (l1 < l2) ? 1.f : ((l1 == l2) ? 0.5f : 0.f);
    const float g = -(w1 * d1 + (1.f - w1) * d2) / float(B);
    const int64_t off = b * T;
    for (int64_t t = tid; t < T; t += kThreads) out_dlogp[off + t] = g * mask[off + t];
}

}  // namespace
}  // namespace trlk

using namespace trlk;

extern "C" int trlk_group_advantages(const float* d_rewards, int64_t n, int32_t group_size, int32_t scale_mode,
                                     float* d_out_advantages, trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(n >= 0, TRLK_ERR_BAD_SHAPE, "group_advantages: n must be >= 0 (got %lld)", (long long)n);
    TRLK_REQUIRE(group_size >= 1, TRLK_ERR_BAD_SHAPE, "group_advantages: group_size must be >= 1 (got %d)", group_size);
    TRLK_REQUIRE(n % group_size == 0, TRLK_ERR_BAD_SHAPE, "group_advantages: n = %lld is not a multiple of group_size = %d",
                 (long long)n, group_size);
    TRLK_REQUIRE(scale_mode >= TRLK_SCALE_GROUP && scale_mode <= TRLK_SCALE_NONE, TRLK_ERR_BAD_VALUE,
                 "group_advantages: unknown scale_mode %d", scale_mode);
    if (n == 0) return TRLK_OK;
    TRLK_REQUIRE(d_rewards != nullptr && d_out_advantages != nullptr, TRLK_ERR_NULL_POINTER,
                 "group_advantages: null pointer");
    hipLaunchKernelGGL(group_advantages_kernel, dim3(1), dim3(kThreads), 0, static_cast<hipStream_t>(stream),
                       d_rewards, n, group_size, scale_mode, d_out_advantages);
    return launch_status("group_advantages");
}

extern "C" size_t trlk_grpo_workspace_bytes(int64_t n_seq) {
    return n_seq > 0 ? size_t(n_seq) * kRowStats * sizeof(float) : 0;
}

namespace {

struct GrpoLossCall {
    const float *d_logp, *d_old_logp, *d_ref_logp, *d_entropy, *d_advantages;
    int64_t adv_stride_b, adv_stride_t;
    const float *d_mask, *d_token_weight, *d_entropy_mask, *d_seq_coef;
    int64_t n_seq, seq_len;
    int32_t loss_type, policy_term, sequence_level;
    float epsilon_low, epsilon_high, delta, beta;
    int32_t use_bias_correction_kl;
    float grad_accum_steps, dr_grpo_denominator;
    const float* d_dapo_normalizer;
    float num_processes, entropy_coef, sapo_temperature_pos, sapo_temperature_neg;
    float *d_out_loss, *d_out_metrics, *d_out_dlogp, *d_out_dentropy;
};

// Argument checks shared by the two GRPO-loss entry points (everything but the workspace).
int grpo_loss_validate(const GrpoLossCall& c) {
    TRLK_REQUIRE(c.n_seq >= 1 && c.seq_len >= 1, TRLK_ERR_BAD_SHAPE, "grpo_loss: need n_seq >= 1 and seq_len >= 1 (got %lld x %lld)",
                 (long long)c.n_seq, (long long)c.seq_len);
    TRLK_REQUIRE(c.n_seq < (int64_t(1) << 31), TRLK_ERR_BAD_SHAPE, "grpo_loss: too many sequences");
    TRLK_REQUIRE(c.loss_type >= TRLK_GRPO && c.loss_type <= TRLK_LUSPO, TRLK_ERR_BAD_VALUE, "grpo_loss: unknown loss_type %d",
                 c.loss_type);
    TRLK_REQUIRE(c.policy_term >= TRLK_TERM_CLIP && c.policy_term <= TRLK_TERM_WEIGHTED_LOGP, TRLK_ERR_BAD_VALUE,
                 "grpo_loss: unknown policy_term %d", c.policy_term);
    TRLK_REQUIRE(c.policy_term != TRLK_TERM_WEIGHTED_LOGP || c.d_seq_coef != nullptr, TRLK_ERR_NULL_POINTER,
                 "grpo_loss: the weighted-logp policy term needs the per-sequence coefficients");
    TRLK_REQUIRE(c.policy_term != TRLK_TERM_SAPO || (c.sapo_temperature_pos > 0.f && c.sapo_temperature_neg > 0.f),
                 TRLK_ERR_BAD_VALUE, "grpo_loss: SAPO temperatures must be positive");
    TRLK_REQUIRE(c.d_logp && c.d_advantages && c.d_mask && c.d_out_loss && c.d_out_metrics && c.d_out_dlogp, TRLK_ERR_NULL_POINTER,
                 "grpo_loss: a required pointer is null");
    TRLK_REQUIRE(c.beta == 0.f || c.d_ref_logp != nullptr, TRLK_ERR_NULL_POINTER,
                 "grpo_loss: beta != 0 needs the reference log-probs");
    TRLK_REQUIRE(c.entropy_coef == 0.f || (c.d_entropy != nullptr && c.d_out_dentropy != nullptr), TRLK_ERR_NULL_POINTER,
                 "grpo_loss: entropy_coef != 0 needs entropy and out_dentropy");
    TRLK_REQUIRE(c.loss_type != TRLK_DAPO || c.d_dapo_normalizer != nullptr, TRLK_ERR_NULL_POINTER,
                 "grpo_loss: the DAPO loss needs the num_items_in_batch device scalar");
    TRLK_REQUIRE(c.loss_type != TRLK_DR_GRPO || c.dr_grpo_denominator > 0.f, TRLK_ERR_BAD_VALUE,
                 "grpo_loss: dr_grpo_denominator must be positive");
    TRLK_REQUIRE(c.grad_accum_steps > 0.f && c.num_processes > 0.f, TRLK_ERR_BAD_VALUE,
                 "grpo_loss: grad_accum_steps and num_processes must be positive");
    TRLK_REQUIRE(c.epsilon_low == c.epsilon_low && c.epsilon_high == c.epsilon_high, TRLK_ERR_BAD_VALUE, "grpo_loss: epsilon is NaN");
    return TRLK_OK;
}

// The two launches of the GRPO loss; `ws` holds kRowStats floats per sequence, all of which the first
// kernel writes before the second reads them (nothing has to be cleared).
int grpo_loss_launch(const GrpoLossCall& c, float* ws, trlk_stream_t stream) {
    // LUSPO's per-token term is one value per sequence only with sequence-level weights, one advantage per
    // sequence, no KL term and no per-token weights; in every other case it is [B, T] and the reference's
    // mean runs over all B * T entries, masked or not
    const int luspo_dense = c.loss_type == TRLK_LUSPO &&
                            !(c.sequence_level && c.beta == 0.f && c.d_token_weight == nullptr && c.adv_stride_t == 0);
    GrpoArgs a{c.d_logp, c.d_old_logp, c.d_ref_logp, c.d_entropy, c.d_advantages, c.d_mask, c.d_token_weight,
               c.d_entropy_mask, c.d_seq_coef, c.adv_stride_b, c.adv_stride_t, c.n_seq, c.seq_len, c.loss_type,
               c.policy_term, c.sequence_level != 0, luspo_dense, c.epsilon_low, c.epsilon_high, c.delta, c.beta,
               c.use_bias_correction_kl, c.grad_accum_steps, c.dr_grpo_denominator, c.d_dapo_normalizer,
               c.num_processes, c.entropy_coef, c.sapo_temperature_pos, c.sapo_temperature_neg, c.d_out_loss,
               c.d_out_metrics, c.d_out_dlogp, c.d_out_dentropy, ws};
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(grpo_rows_kernel, dim3((unsigned)c.n_seq), dim3(kThreads), 0, s, a);
    if (int rc = launch_status("grpo_loss (rows)")) return rc;
    hipLaunchKernelGGL(grpo_finish_kernel, dim3((unsigned)c.n_seq), dim3(kThreads), 0, s, a);
    return launch_status("grpo_loss (finish)");
}

}  // namespace

extern "C" int trlk_grpo_loss(const float* d_logp, const float* d_old_logp, const float* d_ref_logp,
                              const float* d_entropy, const float* d_advantages, int64_t adv_stride_b,
                              int64_t adv_stride_t, const float* d_mask, const float* d_token_weight,
                              const float* d_entropy_mask, const float* d_seq_coef, int64_t n_seq, int64_t seq_len,
                              int32_t loss_type, int32_t policy_term, int32_t sequence_level, float epsilon_low,
                              float epsilon_high, float delta, float beta, int32_t use_bias_correction_kl,
                              float grad_accum_steps, float dr_grpo_denominator, const float* d_dapo_normalizer,
                              float num_processes, float entropy_coef, float sapo_temperature_pos,
                              float sapo_temperature_neg, float* d_out_loss, float* d_out_metrics, float* d_out_dlogp,
                              float* d_out_dentropy, void* d_workspace, size_t workspace_bytes, trlk_stream_t stream) {
    clear_error();
    const GrpoLossCall c{d_logp, d_old_logp, d_ref_logp, d_entropy, d_advantages, adv_stride_b, adv_stride_t, d_mask,
                         d_token_weight, d_entropy_mask, d_seq_coef, n_seq, seq_len, loss_type, policy_term,
                         sequence_level, epsilon_low, epsilon_high, delta, beta, use_bias_correction_kl,
                         grad_accum_steps, dr_grpo_denominator, d_dapo_normalizer, num_processes, entropy_coef,
                         sapo_temperature_pos, sapo_temperature_neg, d_out_loss, d_out_metrics, d_out_dlogp,
                         d_out_dentropy};
    if (int rc = grpo_loss_validate(c)) return rc;
    TRLK_REQUIRE(d_workspace != nullptr && workspace_bytes >= trlk_grpo_workspace_bytes(n_seq), TRLK_ERR_WORKSPACE,
                 "grpo_loss: workspace of %zu bytes needed, %zu given", trlk_grpo_workspace_bytes(n_seq), workspace_bytes);
    return grpo_loss_launch(c, static_cast<float*>(d_workspace), stream);
}

// ---- the GRPO loss for callers that cannot allocate: its per-sequence partial sums live in a file-scope device
// array instead of a caller workspace.  Every GPU the library runs on holds its own copy of the array (at its own
// address) until the process ends; every call on a GPU shares that GPU's copy, so calls that overlap on one GPU
// (two streams, two threads) race.  The array keeps the previous call's contents; nothing needs clearing because
// the first kernel writes every float the second one reads.
constexpr int64_t kStaticMaxSeq = 8192;  // 8192 sequences * 16 floats = 512 KiB per GPU
static __device__ __align__(256) float grpo_static_scratch[kStaticMaxSeq * kRowStats];

namespace {
constexpr int kMaxDevices = 64;
float* g_static_scratch_ptr[kMaxDevices] = {};  // device address of grpo_static_scratch per GPU (0 = not yet asked)
std::mutex g_static_scratch_mutex;

// The array's name is a host-side handle, not a device address: the address on the current device comes from
// hipGetSymbolAddress, once per device, and is what kernels get.
int static_scratch_for_current_device(float** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(int(e), "grpo_loss_static: hipGetDevice failed: %s", hipGetErrorString(e));
    TRLK_REQUIRE(dev >= 0 && dev < kMaxDevices, TRLK_ERR_UNSUPPORTED, "grpo_loss_static: device ordinal %d is out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(grpo_static_scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(e != hipSuccess ? int(e) : int(hipErrorInvalidSymbol), "grpo_loss_static: hipGetSymbolAddress failed: %s",
                        hipGetErrorString(e));
        g_static_scratch_ptr[dev] = static_cast<float*>(p);
    }
    *out = g_static_scratch_ptr[dev];
    return TRLK_OK;
}
}  // namespace

extern "C" int trlk_init(void) {
    clear_error();
    float* p = nullptr;
    if (int rc = static_scratch_for_current_device(&p)) return rc;
    return grpo_fused_reserve_lds();
}

extern "C" int64_t trlk_grpo_loss_static_max_seq(void) { return kStaticMaxSeq; }

extern "C" int trlk_grpo_loss_static(const float* d_logp, const float* d_old_logp, const float* d_ref_logp,
                                     const float* d_entropy, const float* d_advantages, int64_t adv_stride_b,
                                     int64_t adv_stride_t, const float* d_mask, const float* d_token_weight,
                                     const float* d_entropy_mask, const float* d_seq_coef, int64_t n_seq,
                                     int64_t seq_len, int32_t loss_type, int32_t policy_term, int32_t sequence_level,
                                     float epsilon_low, float epsilon_high, float delta, float beta,
                                     int32_t use_bias_correction_kl, float grad_accum_steps, float dr_grpo_denominator,
                                     const float* d_dapo_normalizer, float num_processes, float entropy_coef,
                                     float sapo_temperature_pos, float sapo_temperature_neg, float* d_out_loss,
                                     float* d_out_metrics, float* d_out_dlogp, float* d_out_dentropy,
                                     trlk_stream_t stream) {
    clear_error();
    const GrpoLossCall c{d_logp, d_old_logp, d_ref_logp, d_entropy, d_advantages, adv_stride_b, adv_stride_t, d_mask,
                         d_token_weight, d_entropy_mask, d_seq_coef, n_seq, seq_len, loss_type, policy_term,
                         sequence_level, epsilon_low, epsilon_high, delta, beta, use_bias_correction_kl,
                         grad_accum_steps, dr_grpo_denominator, d_dapo_normalizer, num_processes, entropy_coef,
                         sapo_temperature_pos, sapo_temperature_neg, d_out_loss, d_out_metrics, d_out_dlogp,
                         d_out_dentropy};
    if (int rc = grpo_loss_validate(c)) return rc;
    TRLK_REQUIRE(n_seq <= kStaticMaxSeq, TRLK_ERR_WORKSPACE,
                 "grpo_loss_static: %lld sequences exceed the built-in scratch of %lld; use trlk_grpo_loss with a workspace",
                 (long long)n_seq, (long long)kStaticMaxSeq);
    float* ws = nullptr;
    if (int rc = static_scratch_for_current_device(&ws)) return rc;
    return grpo_loss_launch(c, ws, stream);
}

extern "C" int trlk_dpo_loss(const float* d_token_logp, const float* d_mask, const float* d_ref_chosen,
                             const float* d_ref_rejected, int64_t n_seq, int64_t seq_len, float beta,
                             float* d_out_seq_logps, float* d_out_loss, float* d_out_metrics, float* d_out_dlogp,
                             trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(n_seq >= 2 && n_seq % 2 == 0, TRLK_ERR_BAD_SHAPE,
                 "dpo_loss: n_seq must be even and >= 2 ([chosen; rejected] layout), got %lld", (long long)n_seq);
    TRLK_REQUIRE(seq_len >= 1, TRLK_ERR_BAD_SHAPE, "dpo_loss: seq_len must be >= 1");
    TRLK_REQUIRE(n_seq < (int64_t(1) << 31), TRLK_ERR_BAD_SHAPE, "dpo_loss: too many sequences");
    TRLK_REQUIRE(d_token_logp && d_mask && d_ref_chosen && d_ref_rejected && d_out_seq_logps && d_out_loss &&
                     d_out_metrics && d_out_dlogp,
                 TRLK_ERR_NULL_POINTER, "dpo_loss: a required pointer is null");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(masked_row_sum_kernel<true>, dim3((unsigned)n_seq), dim3(kThreads), 0, s, d_token_logp, d_mask,
                       seq_len, d_out_seq_logps);
    if (int rc = launch_status("dpo_loss (row sums)")) return rc;
    hipLaunchKernelGGL(dpo_finish_kernel, dim3((unsigned)n_seq), dim3(kThreads), 0, s, d_out_seq_logps, d_ref_chosen,
                       d_ref_rejected, d_mask, n_seq, seq_len, beta, d_out_loss, d_out_metrics, d_out_dlogp);
    return launch_status("dpo_loss (finish)");
}

extern "C" int trlk_rloo_loss(const float* d_token_logp, const float* d_mask, const float* d_old_seq_logps,
                              const float* d_advantages, int64_t n_seq, int64_t seq_len, float epsilon_low,
                              float epsilon_high, float* d_out_seq_logps, float* d_out_loss, float* d_out_metrics,
                              float* d_out_dlogp, trlk_stream_t stream) {
    clear_error();
    TRLK_REQUIRE(n_seq >= 1 && seq_len >= 1, TRLK_ERR_BAD_SHAPE, "rloo_loss: need n_seq >= 1 and seq_len >= 1");
    TRLK_REQUIRE(n_seq < (int64_t(1) << 31), TRLK_ERR_BAD_SHAPE, "rloo_loss: too many sequences");
    TRLK_REQUIRE(d_token_logp && d_mask && d_old_seq_logps && d_advantages && d_out_seq_logps && d_out_loss &&
                     d_out_metrics && d_out_dlogp,
                 TRLK_ERR_NULL_POINTER, "rloo_loss: a required pointer is null");
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(masked_row_sum_kernel<false>, dim3((unsigned)n_seq), dim3(kThreads), 0, s, d_token_logp, d_mask,
                       seq_len, d_out_seq_logps);
    if (int rc = launch_status("rloo_loss (row sums)")) return rc;
    hipLaunchKernelGGL(rloo_finish_kernel, dim3((unsigned)n_seq), dim3(kThreads), 0, s, d_out_seq_logps,
                       d_old_seq_logps, d_advantages, d_mask, n_seq, seq_len, epsilon_low, epsilon_high, d_out_loss,
                       d_out_metrics, d_out_dlogp);
    return launch_status("rloo_loss (finish)");
}

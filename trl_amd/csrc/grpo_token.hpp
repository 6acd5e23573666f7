// Per-token arithmetic of the GRPO loss (trl/trainer/grpo_trainer.py:3054-3121), shared by the [B, T]-sized loss
// kernels and by the single-pass kernel that goes from the logits to their gradient.  `Args` is any struct with the
// fields policy_term, eps_low, eps_high, delta, sapo_tau_pos, sapo_tau_neg, beta, bias_kl.
#pragma once

#include "common.hpp"

namespace trlk {

// Policy term f(c, A, logp) of one token (or one sequence) and its two partial derivatives:
// through the log importance ratio ln c, and directly through logp (terms that multiply logp itself).
struct PolicyTerm {
    float f, d_lnc, d_logp, low, high, aux;
};

template <class Args>
__device__ __forceinline__ PolicyTerm policy_term(const Args& a, float c_raw, float A, float lp, float coef) {
    PolicyTerm r{0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const float lo = 1.f - a.eps_low, hi = 1.f + a.eps_high;
    switch (a.policy_term) {
        case TRLK_TERM_CLIP: {  // -min(c' A, clamp(c, lo, hi) A), c' = min(c, delta)   (grpo_trainer.py:3083-3091)
            const bool has_delta = a.delta == a.delta;
            const float c2 = fminf(fmaxf(c_raw, lo), hi);
            const float c1 = has_delta ? fminf(c_raw, a.delta) : c_raw;
            const float l1 = c1 * A, l2 = c2 * A;
            // d c / d ln c = c; clamp passes the gradient on the closed interval
            const float d1 = (!has_delta || c_raw <= a.delta) ? A * c_raw : 0.f;
            const float d2 = (c_raw >= lo && c_raw <= hi) ? A * c_raw : 0.f;
            // min(l1, l2): the gradient goes to the smaller operand, half to each on a tie
            const float w1 = (l1 < l2) ? 1.f : ((l1 == l2) ? 0.5f : 0.f);
            r.f = -fminf(l1, l2);
            r.d_lnc = -(w1 * d1 + (1.f - w1) * d2);
            r.low = (c1 < lo && A < 0.f) ? 1.f : 0.f;
            r.high = (c1 > hi && A > 0.f) ? 1.f : 0.f;
            break;
        }
        case TRLK_TERM_CISPO: {  // -min(c, eps_high).detach() * A * logp   (:3080-3082)
            const float cl = fminf(c_raw, a.eps_high);
            r.f = -cl * A * lp;
            r.d_logp = -cl * A;
            r.aux = (c_raw > a.eps_high && A > 0.f) ? 1.f : 0.f;
            break;
        }
        case TRLK_TERM_SAPO: {  // -sigmoid(tau (c - 1)) * 4 / tau * A   (:3092-3095)
            const float tau = A > 0.f ? a.sapo_tau_pos : a.sapo_tau_neg;
            const float sg = 1.f / (1.f + expf(-tau * (c_raw - 1.f)));
            r.f = -sg * 4.f / tau * A;
            r.d_lnc = -4.f * A * sg * (1.f - sg) * c_raw;
            break;
        }
        default: {  // TRLK_TERM_WEIGHTED_LOGP: -coef * A * logp with a given, detached per-sequence coef (:3096-3107)
            r.f = -coef * A * lp;
            r.d_logp = -coef * A;
            r.aux = coef;
            break;
        }
    }
    return r;
}

// Loss term of one token before mask and normalisation, `pl`, its KL part `kl`, and the derivatives of `pl`
// through the log importance ratio (`g_lnc`) and directly through the log-prob (`g_lp`).  `w` is the token's
// weight (1 without one), `ref_lp` is read only when beta != 0.
template <class Args>
__device__ __forceinline__ void grpo_token_terms(const Args& a, const PolicyTerm& p, float c_raw, float lp, float w,
                                                 float ref_lp, float& pl, float& kl, float& g_lnc, float& g_lp) {
    pl = p.f * w;
    g_lnc = p.d_lnc * w;
    g_lp = p.d_logp * w;
    kl = 0.f;
    if (a.beta != 0.f) {  // k3 estimator exp(d) - d - 1, d = ref - logp   (:3069-3076)
        const float d = ref_lp - lp;
        const float e = expf(d);
        kl = e - d - 1.f;
        float dkl = 1.f - e;
        if (a.bias_kl) {  // kl * c: the factor c is differentiated through ln c
            g_lnc += a.beta * kl * c_raw;
            dkl *= c_raw;
            kl *= c_raw;
        }
        pl += a.beta * kl;
        g_lp += a.beta * dkl;
    }
}

}  // namespace trlk

// Per-token arithmetic of the clipped policy-gradient loss, shared by the stand-alone loss kernel
// and by the kernel that fuses it into the logits pass.  fp32 like the PyTorch ops it mirrors.
#pragma once

#include <float.h>
#include <math.h>

#include "common.hpp"

namespace nrl {

// per-row partial slots
enum {
    P_ACTOR = 0, P_KL, P_MULT_ERR, P_GEN_KL, P_POLICY_KL, P_JS, P_SAMPLING, P_ENTROPY, P_RATIO, P_RATIO_CL,
    P_OOB, P_NLL, P_N_CORRECT, P_N_SELECTED, P_SAMPLE_MASK, P_SEQ_W, P_R_MIN, P_R_MAX, P_RC_MIN, P_RC_MAX,
    P_COUNT
};

struct GrpoArgs {
    nrl_grpo_cfg cfg;
    nrl_grpo_inputs in;
    float* dlp;
    float* dlpu;
    double* parts;  // [B, P_COUNT]
};

// per-sequence quantities the token terms depend on
struct SeqStats {
    float seq_den;    // sum(token_mask) + 1e-8
    float seq_ratio;  // GSPO: exp(masked mean of lp - prev)
    float seq_w;      // sequence-level importance weight
    float seq_keep;   // seq-mask-tis: 1 if the sequence's geometric-mean IS ratio is inside the bounds
};

struct TokenIn {
    float lp, lpu, prev, gen, ref, adv, tm, smv, correct;
    float den_t, den_s;
};

struct TokenOut {
    float term[P_SAMPLE_MASK];  // contributions to the per-token partial sums (slots below P_SAMPLE_MASK)
    float ratio, ratio_cl;
    float d_actor;  // d loss / d lp through the surrogate (GSPO: through the sequence ratio, before the chain rule)
    float d_lpu;    // d loss / d (unfiltered) lp through the KL term
    bool selected;  // mask != 0
};

__device__ __forceinline__ float finite_or_zero(float x) { return (x - x == 0.f) ? x : 0.f; }

__device__ __forceinline__ float kl_value(int type, float logr) {
    if (type == 1) return -logr;
    if (type == 2) return (logr * logr) / 2.f;
    return (expf(logr) - 1.f) - logr;
}

// d kl / d logr
__device__ __forceinline__ float kl_slope(int type, float logr) {
    if (type == 1) return -1.f;
    if (type == 2) return logr;
    return expf(logr) - 1.f;
}

__device__ __forceinline__ float clampf(float x, float lo, float hi) {
    // torch.clamp: min(max(x, lo), hi) with NaN propagating
    if (x != x) return x;
    return fminf(fmaxf(x, lo), hi);
}

// gradient share of the larger (or, for SMALLER, the smaller) of two values: 1, 1/2 on a tie, 0
__device__ __forceinline__ float pick_weight(float self, float other, bool want_max) {
    if (self == other) return 0.5f;
    return (want_max ? self > other : self < other) ? 1.f : 0.f;
}

template <bool GSPO>
__device__ __forceinline__ TokenOut token_eval(const nrl_grpo_cfg& c, const SeqStats& st, const TokenIn& ti) {
    TokenOut o;
#pragma unroll
    for (int k = 0; k < P_SAMPLE_MASK; ++k) o.term[k] = 0.f;
    const float lp = ti.lp, lpu = ti.lpu, prev = ti.prev, gen = ti.gen, adv = ti.adv, tm = ti.tm, smv = ti.smv;
    const float seq_den = st.seq_den, seq_ratio = st.seq_ratio, seq_w = st.seq_w, seq_keep = st.seq_keep;
    const float den_t = ti.den_t, den_s = ti.den_s, correct = ti.correct;
    const float tis_floor = c.tis_min;  // the host passes 0 when the lower bound is unset
    const float clip_lo = 1.0f - c.ratio_clip_min, clip_hi = 1.0f + c.ratio_clip_max;
    float* acc = o.term;
    {
        const float mask = tm * smv;
        // gradient coefficient of a per-token value in the reduced loss
        const float coef = c.token_level_loss ? mask / den_t : (tm / seq_den) * (smv / den_s);

        // ---- diagnostics on (gen, prev) ----
        acc[P_MULT_ERR] += expf(fabsf(gen - prev) * mask) * mask;
        acc[P_GEN_KL] += kl_value(c.kl_type, prev - gen) * mask;
        acc[P_POLICY_KL] += kl_value(c.kl_type, gen - prev) * mask;
        {
            const float log_mix = logf(0.5f * expf(prev) + 0.5f * expf(gen));
            const float dp = prev - log_mix, dg = gen - log_mix;
            const float kp = (expf(dp) - dp) - 1.f, kg = (expf(dg) - dg) - 1.f;
            acc[P_JS] += (0.5f * kp + 0.5f * kg) * mask;
        }

        // ---- KL to the reference policy ----
        float d_lpu = 0.f;
        if (c.has_kl) {
            const float ref = ti.ref;
            const float w_raw = c.use_on_policy_kl_approximation ? expf(lpu - gen) : expf(lpu - lpu);
            const float w = finite_or_zero(w_raw);
            float w_slope = w;  // d w / d lpu (zero where nan_to_num replaced the value)
            float logr = ref - lpu;
            float in_range = 1.f;
            if (c.has_kl_input_clamp) {
                const float cl = clampf(logr, -c.kl_input_clamp, c.kl_input_clamp);
                if (!(logr == cl)) { w_slope = 0.f; in_range = 0.f; }
                logr = cl;
            }
            const float k = kl_value(c.kl_type, logr);
            float v = w * k;
            // d v / d lpu: weight term + kl term (d logr / d lpu = -1)
            float dv = w_slope * k + w * (-kl_slope(c.kl_type, logr)) * in_range;
            if (c.has_kl_output_clamp) {
                const float vc = clampf(v, -c.kl_output_clamp, c.kl_output_clamp);
                if (!(v >= -c.kl_output_clamp && v <= c.kl_output_clamp)) dv = 0.f;
                v = vc;
            }
            const float klt = c.kl_beta * v;
            acc[P_KL] += c.token_level_loss ? klt * mask : (klt * tm);
            d_lpu = coef * (c.kl_beta * dv);
        }

        // ---- probability ratio and clipped surrogate ----
        float ratio, ratio_cl, d_clip;  // d_clip = d clip_loss / d lp (non-GSPO) or / d ratio (GSPO)
        float clip;
        if (c.force_on_policy_ratio) {
            ratio = expf(lp - lp);
            ratio_cl = ratio;
            clip = nan_max(-adv * ratio, -adv * ratio_cl);
            d_clip = -adv * ratio;
        } else if (!c.disable_ppo_ratio) {
            ratio = GSPO ? seq_ratio : expf(lp - prev);
            ratio_cl = clampf(ratio, clip_lo, clip_hi);
            if (c.use_cispo) {
                clip = -adv * ratio_cl * lp;
                d_clip = -adv * ratio_cl;
            } else {
                const float l1 = -adv * ratio, l2 = -adv * ratio_cl;
                clip = nan_max(l1, l2);
                const float inside = (ratio >= clip_lo && ratio <= clip_hi) ? 1.f : 0.f;
                const float share = pick_weight(l1, l2, true) + pick_weight(l2, l1, true) * inside;
                d_clip = -adv * share * (GSPO ? 1.f : ratio);
            }
        } else {
            ratio = lp;
            ratio_cl = lp;
            clip = nan_max(-adv * ratio, -adv * ratio_cl);
            d_clip = -adv;
        }
        if (c.has_dual_clip) {
            const float l3 = -adv * c.ratio_clip_c;
            if (adv < 0.f) {
                d_clip *= pick_weight(clip, l3, false);
                clip = nan_min(clip, l3);
            }
        }

        // ---- off-policy importance weight ----
        float w_is = c.sequence_level_importance_ratios ? seq_w : finite_or_zero(expf(prev - gen));
        if (c.tis_type == NRL_TIS_TIS) {
            acc[P_OOB] += ((w_is > c.tis_max || w_is < tis_floor) ? 1.f : 0.f) * mask;
            w_is = clampf(w_is, tis_floor, c.tis_max);
        } else if (c.tis_type == NRL_TIS_ICEPOP) {
            const bool kept = w_is >= c.tis_min && w_is <= c.tis_max;
            acc[P_OOB] += (kept ? 0.f : 1.f) * mask;
            w_is = kept ? w_is : 0.f;
        } else if (c.tis_type == NRL_TIS_SEQ_MASK) {
            w_is = w_is * seq_keep;
        }
        const float w_use = c.use_importance_sampling_correction ? w_is : 1.f;

        const float actor_t = w_use * clip;
        acc[P_ACTOR] += c.token_level_loss ? actor_t * mask : actor_t * tm;
        if (!c.sequence_level_importance_ratios) acc[P_SAMPLING] += w_is * mask;
        acc[P_ENTROPY] += (expf(lp - gen) * lp) * mask;
        acc[P_RATIO] += ratio * mask;
        acc[P_RATIO_CL] += ratio_cl * mask;
        if (c.has_nll) {
            const float cm = mask * correct;
            acc[P_NLL] += (-lp) * cm;
            acc[P_N_CORRECT] += cm;
        }
        if (mask != 0.f) {
            acc[P_N_SELECTED] += 1.f;
        }

        o.ratio = ratio;
        o.ratio_cl = ratio_cl;
        o.selected = mask != 0.f;
        o.d_actor = coef * w_use * d_clip;
        o.d_lpu = d_lpu;
    }
    return o;
}

}  // namespace nrl

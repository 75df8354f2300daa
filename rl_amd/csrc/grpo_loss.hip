// K4: clipped policy-gradient (GRPO family) loss, its gradient with respect to the token
// logprobs and all metrics, fused.
//
// Launch 1 (one workgroup per sequence row): per-row statistics that the sequence-level modes
// need (token count, mean log-ratio, summed IS log-weight), then every per-token term - ratio,
// clip / dual clip / CISPO, k1-k3 KL with its clamps and importance weight, truncated IS - with
// the analytic gradient written straight to dlp, and per-row partial sums of the loss and of
// every diagnostic in float64.  Launch 2 (one workgroup): fixed-order reduction of the row
// partials, normalisation, and the metrics record the host reads back with a single copy.
// Token arithmetic is fp32 like the PyTorch ops it replaces; only the accumulations are wider.
//
// The data are [B, S-1] fp32 arrays (a few tens of bytes per token), so this stage is launch-
// latency bound; it exists to remove ~40 small kernels and ~15 device->host syncs per call.

#include <float.h>
#include <math.h>

#include "common.hpp"

namespace nrl {

constexpr int kLossBlock = 256;
constexpr int kLossWaves = kLossBlock / kWave;

// per-row partial slots
enum {
    P_ACTOR = 0, P_KL, P_MULT_ERR, P_GEN_KL, P_POLICY_KL, P_JS, P_SAMPLING, P_ENTROPY, P_RATIO, P_RATIO_CL,
    P_OOB, P_NLL, P_N_CORRECT, P_SAMPLE_MASK, P_N_SELECTED, P_SEQ_W, P_R_MIN, P_R_MAX, P_RC_MIN, P_RC_MAX,
    P_COUNT
};

struct GrpoArgs {
    nrl_grpo_cfg cfg;
    nrl_grpo_inputs in;
    float* dlp;
    float* dlpu;
    double* parts;  // [B, P_COUNT]
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
__global__ __launch_bounds__(kLossBlock) void grpo_rows_kernel(GrpoArgs a) {
    __shared__ double sm_d[kLossWaves];
    __shared__ float sm_f[kLossWaves];
    const nrl_grpo_cfg& c = a.cfg;
    const nrl_grpo_inputs& in = a.in;
    const int64_t b = blockIdx.x;
    const int tid = threadIdx.x;
    const int64_t n = in.sm1;

    const float* lp_row = in.lp + b * in.lp_stride;
    const float* lpu_row = in.lpu ? in.lpu + b * in.lpu_stride : lp_row;
    const float* prev_row = c.force_on_policy_ratio ? lp_row : in.prev + b * in.prev_stride;
    const float* gen_row = in.gen + b * in.gen_stride;
    const float* ref_row = c.has_kl ? in.ref + b * in.ref_stride : nullptr;
    const float* adv_row = in.adv + b * in.adv_stride;
    const float* tm_row = in.token_mask + b * in.token_mask_stride;
    const float smv = in.sample_mask[b];
    const float correct = c.has_nll ? in.correct_mask[b] : 0.f;
    const float den_s = in.global_valid[0] + 1e-8f;
    const float den_t = in.global_valid[1] + 1e-8f;

    // ---- row statistics ----
    double s_tm = 0, s_lr = 0, s_is = 0, s_geo = 0;
    for (int64_t t = tid; t < n; t += kLossBlock) {
        const float tm = tm_row[t];
        const float prev = prev_row[t], gen = gen_row[t];
        s_tm += tm;
        s_lr += (lp_row[t] - prev) * tm;
        s_is += (prev - gen) * (tm * smv);
        s_geo += finite_or_zero(prev - gen) * tm;
    }
    const float n_tm = static_cast<float>(block_sum<double, kLossWaves>(s_tm, sm_d));
    const float seq_den = n_tm + 1e-8f;
    float seq_ratio = 1.f, seq_w = 1.f, seq_keep = 1.f;
    if (GSPO) seq_ratio = expf(static_cast<float>(block_sum<double, kLossWaves>(s_lr, sm_d)) / seq_den);
    if (c.sequence_level_importance_ratios)
        seq_w = finite_or_zero(expf(static_cast<float>(block_sum<double, kLossWaves>(s_is, sm_d))));
    if (c.tis_type == NRL_TIS_SEQ_MASK) {
        const float geo = expf(static_cast<float>(block_sum<double, kLossWaves>(s_geo, sm_d)) / seq_den);
        seq_keep = (geo >= c.tis_min && geo <= c.tis_max) ? 1.f : 0.f;
    }
    const float tis_floor = c.tis_min;  // host passes 0 when the lower bound is unset

    const float clip_lo = 1.0f - c.ratio_clip_min, clip_hi = 1.0f + c.ratio_clip_max;

    double acc[P_R_MIN];
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) acc[k] = 0;
    float r_min = INFINITY, r_max = -INFINITY, rc_min = INFINITY, rc_max = -INFINITY;
    double gspo_k = 0;  // sum_t coef * w * d clip / d ratio  (GSPO only)

    for (int64_t t = tid; t < n; t += kLossBlock) {
        const float lp = lp_row[t], lpu = lpu_row[t], prev = prev_row[t], gen = gen_row[t];
        const float adv = adv_row[t], tm = tm_row[t];
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
            const float ref = ref_row[t];
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
            acc[P_N_SELECTED] += 1.0;
            r_min = fminf(r_min, ratio); r_max = fmaxf(r_max, ratio);
            rc_min = fminf(rc_min, ratio_cl); rc_max = fmaxf(rc_max, ratio_cl);
        }

        // ---- gradient ----
        const float d_actor = coef * w_use * d_clip;
        if (GSPO) {
            gspo_k += d_actor;
            if (a.dlpu) a.dlpu[b * n + t] = d_lpu;
            else a.dlp[b * n + t] = d_lpu;  // KL share; the ratio share is added below
        } else if (a.dlpu) {
            a.dlp[b * n + t] = d_actor;
            a.dlpu[b * n + t] = d_lpu;
        } else {
            a.dlp[b * n + t] = d_actor + d_lpu;
        }
    }

    if (GSPO) {
        // d ratio_b / d lp[b, s] = ratio_b * tm[b, s] / (n_tm + 1e-8)
        const float k_tot = static_cast<float>(block_sum<double, kLossWaves>(gspo_k, sm_d));
        for (int64_t t = tid; t < n; t += kLossBlock) {
            const float share = k_tot * seq_ratio * (tm_row[t] / seq_den);
            if (a.dlpu) a.dlp[b * n + t] = share;
            else a.dlp[b * n + t] += share;
        }
    }

    // ---- row partials ----
    double* out = a.parts + b * P_COUNT;
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) {
        const double tot = block_sum<double, kLossWaves>(acc[k], sm_d);
        if (tid == 0) out[k] = tot;
    }
    const float mn = block_min<kLossWaves>(r_min, sm_f), mx = block_max<kLossWaves>(r_max, sm_f);
    const float cmn = block_min<kLossWaves>(rc_min, sm_f), cmx = block_max<kLossWaves>(rc_max, sm_f);
    if (tid == 0) {
        if (!c.token_level_loss) {  // sequence-level: masked mean over tokens, then weight by sample_mask
            out[P_ACTOR] = static_cast<double>(static_cast<float>(out[P_ACTOR]) / seq_den) * smv;
            out[P_KL] = static_cast<double>(static_cast<float>(out[P_KL]) / seq_den) * smv;
        }
        out[P_SAMPLE_MASK] = smv;
        out[P_SEQ_W] = c.tis_type == NRL_TIS_SEQ_MASK ? seq_w * seq_keep : seq_w;
        if (c.sequence_level_importance_ratios && c.tis_type == NRL_TIS_TIS) out[P_SEQ_W] = clampf(seq_w, tis_floor, c.tis_max);
        if (c.sequence_level_importance_ratios && c.tis_type == NRL_TIS_ICEPOP)
            out[P_SEQ_W] = (seq_w >= c.tis_min && seq_w <= c.tis_max) ? seq_w : 0.f;
        if (c.tis_type == NRL_TIS_SEQ_MASK) out[P_OOB] = (1.f - seq_keep) * smv;
        out[P_R_MIN] = mn; out[P_R_MAX] = mx; out[P_RC_MIN] = cmn; out[P_RC_MAX] = cmx;
    }
}

// Fixed-order reduction of the row partials and normalisation into the metrics record.
__global__ __launch_bounds__(kLossBlock) void grpo_finish_kernel(GrpoArgs a, float* loss_out, float* metrics) {
    __shared__ double sm_d[kLossWaves];
    __shared__ float sm_f[kLossWaves];
    const nrl_grpo_cfg& c = a.cfg;
    const int tid = threadIdx.x;
    const int64_t nb = a.in.batch;
    double tot[P_R_MIN];
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) tot[k] = 0;
    float r_min = INFINITY, r_max = -INFINITY, rc_min = INFINITY, rc_max = -INFINITY;
    for (int64_t b = tid; b < nb; b += kLossBlock) {
        const double* p = a.parts + b * P_COUNT;
#pragma unroll
        for (int k = 0; k < P_R_MIN; ++k) tot[k] += p[k];
        r_min = fminf(r_min, (float)p[P_R_MIN]); r_max = fmaxf(r_max, (float)p[P_R_MAX]);
        rc_min = fminf(rc_min, (float)p[P_RC_MIN]); rc_max = fmaxf(rc_max, (float)p[P_RC_MAX]);
    }
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) tot[k] = block_sum<double, kLossWaves>(tot[k], sm_d);
    r_min = block_min<kLossWaves>(r_min, sm_f); r_max = block_max<kLossWaves>(r_max, sm_f);
    rc_min = block_min<kLossWaves>(rc_min, sm_f); rc_max = block_max<kLossWaves>(rc_max, sm_f);
    if (tid != 0) return;

    const double den_s = a.in.global_valid[0] + 1e-8f, den_t = a.in.global_valid[1] + 1e-8f;
    const double den_loss = c.token_level_loss ? den_t : den_s;
    const float actor = static_cast<float>(tot[P_ACTOR] / den_loss);
    const float kl = c.has_kl ? static_cast<float>(tot[P_KL] / den_loss) : 0.f;
    float nll = 0.f;
    if (c.has_nll && tot[P_N_CORRECT] > 0) nll = static_cast<float>(tot[P_NLL] / (static_cast<float>(tot[P_N_CORRECT]) + 1e-8f));
    const float loss = (actor + kl) + c.nll_weight * nll;
    loss_out[0] = loss;
    for (int k = 0; k < NRL_GRPO_N_METRICS; ++k) metrics[k] = 0.f;
    metrics[NRL_M_LOSS] = loss;
    metrics[NRL_M_ACTOR_LOSS] = actor;
    metrics[NRL_M_KL] = kl;
    metrics[NRL_M_PROBS_RATIO] = static_cast<float>(tot[P_RATIO] / den_t);
    metrics[NRL_M_PROBS_RATIO_CLAMPED] = static_cast<float>(tot[P_RATIO_CL] / den_t);
    metrics[NRL_M_PROBS_RATIO_MIN] = r_min;
    metrics[NRL_M_PROBS_RATIO_MAX] = r_max;
    metrics[NRL_M_PROBS_RATIO_CLAMPED_MIN] = rc_min;
    metrics[NRL_M_PROBS_RATIO_CLAMPED_MAX] = rc_max;
    metrics[NRL_M_TOKEN_MULT_PROB_ERROR] = static_cast<float>(tot[P_MULT_ERR] / den_t);
    metrics[NRL_M_GEN_KL_ERROR] = static_cast<float>(tot[P_GEN_KL] / den_t);
    metrics[NRL_M_POLICY_KL_ERROR] = static_cast<float>(tot[P_POLICY_KL] / den_t);
    metrics[NRL_M_JS_DIVERGENCE_ERROR] = static_cast<float>(tot[P_JS] / den_t);
    // sequence-level weights: the reference multiplies a [B,1] weight by a [B] mask, which
    // broadcasts to [B,B]; the sum is (sum of weights) * (sum of sample_mask)
    metrics[NRL_M_SAMPLING_IMPORTANCE_RATIO] =
        c.sequence_level_importance_ratios ? static_cast<float>(tot[P_SEQ_W] * tot[P_SAMPLE_MASK] / den_s)
                                           : static_cast<float>(tot[P_SAMPLING] / den_t);
    metrics[NRL_M_NUM_VALID_SAMPLES] = static_cast<float>(tot[P_SAMPLE_MASK]);
    metrics[NRL_M_APPROX_ENTROPY] = -static_cast<float>(tot[P_ENTROPY] / den_t);
    metrics[NRL_M_IS_OOB_RATIO] = static_cast<float>(tot[P_OOB] / (c.tis_type == NRL_TIS_SEQ_MASK ? den_s : den_t));
    metrics[NRL_M_POSITIVE_NLL_LOSS] = nll;
    metrics[NRL_M_N_MASKED_TOKENS] = static_cast<float>(tot[P_N_SELECTED]);
}

// positive-example NLL: d loss / d lp += -weight * mask * correct / (n_correct + 1e-8)
__global__ void grpo_nll_grad_kernel(GrpoArgs a) {
    const int64_t n = a.in.sm1, total = a.in.batch * n;
    double n_correct = 0;
    for (int64_t b = 0; b < a.in.batch; ++b) n_correct += a.parts[b * P_COUNT + P_N_CORRECT];
    if (!(n_correct > 0)) return;
    const float den = static_cast<float>(n_correct) + 1e-8f;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t b = i / n, t = i - b * n;
        const float cm = a.in.token_mask[b * a.in.token_mask_stride + t] * a.in.sample_mask[b] * a.in.correct_mask[b];
        a.dlp[i] += a.cfg.nll_weight * (-(cm / den));
    }
}

// NLLLossFn: one workgroup per row for the partial sums, then the same finish pattern
__global__ __launch_bounds__(kLossBlock) void nll_rows_kernel(nrl_grpo_inputs in, float* dlp, double* parts) {
    __shared__ double sm_d[kLossWaves];
    const int64_t b = blockIdx.x, n = in.sm1;
    const float smv = in.sample_mask[b];
    const float den_t = in.global_valid[1] + 1e-8f;
    double s = 0, cnt = 0;
    for (int64_t t = threadIdx.x; t < n; t += kLossBlock) {
        const float mask = in.token_mask[b * in.token_mask_stride + t] * smv;
        s += in.lp[b * in.lp_stride + t] * mask;
        cnt += mask;
        dlp[b * n + t] = -(mask / den_t);
    }
    s = block_sum<double, kLossWaves>(s, sm_d);
    cnt = block_sum<double, kLossWaves>(cnt, sm_d);
    if (threadIdx.x == 0) { parts[b * 3] = s; parts[b * 3 + 1] = cnt; parts[b * 3 + 2] = smv; }
}

__global__ __launch_bounds__(kLossBlock) void nll_finish_kernel(nrl_grpo_inputs in, const double* parts, float* loss_out,
                                                               float* metrics) {
    __shared__ double sm_d[kLossWaves];
    double s = 0, cnt = 0, smv = 0;
    for (int64_t b = threadIdx.x; b < in.batch; b += kLossBlock) { s += parts[b * 3]; cnt += parts[b * 3 + 1]; smv += parts[b * 3 + 2]; }
    s = block_sum<double, kLossWaves>(s, sm_d);
    cnt = block_sum<double, kLossWaves>(cnt, sm_d);
    smv = block_sum<double, kLossWaves>(smv, sm_d);
    if (threadIdx.x == 0) {
        const double den_t = in.global_valid[1] + 1e-8f;
        const float loss = -static_cast<float>(s / den_t);
        loss_out[0] = loss;
        metrics[0] = loss; metrics[1] = static_cast<float>(cnt); metrics[2] = static_cast<float>(smv);
    }
}

static int check_inputs(const nrl_grpo_inputs* in, bool need_prev, bool need_ref, bool need_adv) {
    if (!in) return fail(NRL_E_INVALID, "inputs is NULL");
    if (in->batch < 0 || in->sm1 < 0) return fail(NRL_E_INVALID, "bad shape [%lld, %lld]", (long long)in->batch, (long long)in->sm1);
    if (in->batch >= (1ll << 31)) return fail(NRL_E_INVALID, "batch too large");
    if (in->batch * in->sm1 == 0) return NRL_OK;
    if (!in->lp || !in->token_mask || !in->sample_mask || !in->global_valid) return fail(NRL_E_INVALID, "null lp, token_mask, sample_mask or global_valid");
    if (need_adv && (!in->gen || !in->adv)) return fail(NRL_E_INVALID, "null generation_logprobs or advantages");
    if (need_prev && !in->prev) return fail(NRL_E_INVALID, "prev_logprobs is NULL");
    if (need_ref && !in->ref) return fail(NRL_E_INVALID, "reference_policy_logprobs is NULL");
    return NRL_OK;
}

}  // namespace nrl

using namespace nrl;

extern "C" int64_t nrl_grpo_loss_workspace_bytes(int64_t batch) {
    return (batch < 1 ? 1 : batch) * P_COUNT * static_cast<int64_t>(sizeof(double));
}

extern "C" int nrl_grpo_loss_fwd_bwd(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float* loss_out, float* dlp_out,
                                     float* dlpu_out, float* metrics_out, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
    if (!cfg) return fail(NRL_E_INVALID, "cfg is NULL");
    if (int e = check_inputs(in, !cfg->force_on_policy_ratio, cfg->has_kl != 0, true)) return e;
    if (cfg->kl_type < 1 || cfg->kl_type > 3) return fail(NRL_E_INVALID, "kl_type must be 1, 2 or 3");
    if (cfg->tis_type < 0 || cfg->tis_type > 3) return fail(NRL_E_INVALID, "bad tis_type");
    if (cfg->sequence_level_importance_ratios && cfg->token_level_loss)
        return fail(NRL_E_INVALID, "sequence-level importance ratios need a sequence-level loss");
    if (cfg->has_nll && !in->correct_mask) return fail(NRL_E_INVALID, "correct_mask is NULL");
    if (!loss_out || !metrics_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (workspace_bytes < nrl_grpo_loss_workspace_bytes(in->batch)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 7) return fail(NRL_E_INVALID, "workspace must be 8-byte aligned");
    const bool split = in->lpu != nullptr && cfg->has_kl;
    if (in->batch * in->sm1 > 0 && (!dlp_out || (split && !dlpu_out))) return fail(NRL_E_INVALID, "null gradient output");
    GrpoArgs a;
    a.cfg = *cfg;
    a.in = *in;
    if (!cfg->has_kl) a.in.lpu = nullptr;
    a.dlp = dlp_out;
    a.dlpu = split ? dlpu_out : nullptr;
    a.parts = static_cast<double*>(workspace);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (in->batch > 0) {
        const bool gspo = cfg->sequence_level_importance_ratios && !cfg->disable_ppo_ratio && !cfg->force_on_policy_ratio;
        if (gspo) grpo_rows_kernel<true><<<dim3((unsigned)in->batch), dim3(kLossBlock), 0, s>>>(a);
        else grpo_rows_kernel<false><<<dim3((unsigned)in->batch), dim3(kLossBlock), 0, s>>>(a);
    }
    grpo_finish_kernel<<<dim3(1), dim3(kLossBlock), 0, s>>>(a, loss_out, metrics_out);
    if (cfg->has_nll && in->batch * in->sm1 > 0) {
        const int64_t total = in->batch * in->sm1;
        const unsigned blocks = (unsigned)((total + 255) / 256 > 1024 ? 1024 : (total + 255) / 256);
        grpo_nll_grad_kernel<<<dim3(blocks), dim3(256), 0, s>>>(a);
    }
    return check_launch("grpo_loss_fwd_bwd");
}

extern "C" int nrl_nll_loss_fwd_bwd(const nrl_grpo_inputs* in, float* loss_out, float* dlp_out, float* metrics_out,
                                    void* workspace, int64_t workspace_bytes, void* stream) {
    if (int e = check_inputs(in, false, false, false)) return e;
    if (!loss_out || !metrics_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (workspace_bytes < nrl_grpo_loss_workspace_bytes(in->batch)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (in->batch * in->sm1 > 0 && !dlp_out) return fail(NRL_E_INVALID, "null gradient output");
    hipStream_t s = static_cast<hipStream_t>(stream);
    double* parts = static_cast<double*>(workspace);
    if (in->batch > 0) nll_rows_kernel<<<dim3((unsigned)in->batch), dim3(kLossBlock), 0, s>>>(*in, dlp_out, parts);
    nll_finish_kernel<<<dim3(1), dim3(kLossBlock), 0, s>>>(*in, parts, loss_out, metrics_out);
    return check_launch("nll_loss_fwd_bwd");
}

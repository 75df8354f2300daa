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

#include <mutex>

#include "common.hpp"
#include "grpo_token.hpp"

namespace nrl {

constexpr int kLossBlock = 256;
constexpr int kLossWaves = kLossBlock / kWave;

// Workgroup-wide reduction of one sequence's accumulators into its row of partials.
__device__ __forceinline__ void store_row_parts(const nrl_grpo_cfg& c, double* out, double (&acc)[P_R_MIN], float r_min,
                                                float r_max, float rc_min, float rc_max, const SeqStats& st, float smv,
                                                double* sm_d, float* sm_f) {
    const int tid = threadIdx.x;
    const float tis_floor = c.tis_min;
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) {
        const double tot = block_sum<double, kLossWaves>(acc[k], sm_d);
        if (tid == 0) out[k] = tot;
    }
    const float mn = block_min<kLossWaves>(r_min, sm_f), mx = block_max<kLossWaves>(r_max, sm_f);
    const float cmn = block_min<kLossWaves>(rc_min, sm_f), cmx = block_max<kLossWaves>(rc_max, sm_f);
    if (tid == 0) {
        const float seq_w = st.seq_w, seq_keep = st.seq_keep;
        if (!c.token_level_loss) {  // sequence-level: masked mean over tokens, then weight by sample_mask
            out[P_ACTOR] = static_cast<double>(static_cast<float>(out[P_ACTOR]) / st.seq_den) * smv;
            out[P_KL] = static_cast<double>(static_cast<float>(out[P_KL]) / st.seq_den) * smv;
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
    double acc[P_R_MIN];
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) acc[k] = 0;
    float r_min = INFINITY, r_max = -INFINITY, rc_min = INFINITY, rc_max = -INFINITY;
    double gspo_k = 0;  // sum_t coef * w * d clip / d ratio  (GSPO only)

    SeqStats st;
    st.seq_den = seq_den; st.seq_ratio = seq_ratio; st.seq_w = seq_w; st.seq_keep = seq_keep;
    for (int64_t t = tid; t < n; t += kLossBlock) {
        TokenIn ti;
        ti.lp = lp_row[t]; ti.lpu = lpu_row[t]; ti.prev = prev_row[t]; ti.gen = gen_row[t];
        ti.ref = c.has_kl ? ref_row[t] : 0.f; ti.adv = adv_row[t]; ti.tm = tm_row[t]; ti.smv = smv; ti.correct = correct;
        ti.den_t = den_t; ti.den_s = den_s;
        const TokenOut o = token_eval<GSPO>(c, st, ti);
#pragma unroll
        for (int k = 0; k < P_SAMPLE_MASK; ++k) acc[k] += o.term[k];
        if (o.selected) {
            r_min = fminf(r_min, o.ratio); r_max = fmaxf(r_max, o.ratio);
            rc_min = fminf(rc_min, o.ratio_cl); rc_max = fmaxf(rc_max, o.ratio_cl);
        }
        const float d_actor = o.d_actor, d_lpu = o.d_lpu;
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

    store_row_parts(c, a.parts + b * P_COUNT, acc, r_min, r_max, rc_min, rc_max, st, smv, sm_d, sm_f);
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

// ---------------------------------------------------------------------------------------------
// Fused pass: logits row -> log-sum-exp -> token logprob -> loss terms and d loss / d logprob ->
// dlogits, with the row held on chip (registers plus an LDS slice) between the reduction and the
// gradient, so the logits are read once and the gradient written once (2 * V * sizeof(logit) per
// token instead of 3).  Valid when d loss / d logprob of a token depends only on that token and on
// per-sequence quantities that do not involve the current logprobs: everything except sequence-level
// probability ratios (GSPO) and the positive-example NLL term.  Tokens whose mask is zero are not
// evaluated: their gradient row is zero-filled without reading the logits and their logprob is
// reported as 0.
// ---------------------------------------------------------------------------------------------
constexpr int kFusedBlock = 1024;
constexpr int kFusedWaves = kFusedBlock / kWave;
constexpr int kFusedMaxRegVec = 16;  // at most 16 16-byte vectors per lane held in registers ...
constexpr int kFusedLdsVec = 4;      // ... and 4 in LDS (64 KiB per workgroup)
constexpr int kFusedMaxVec = kFusedMaxRegVec + kFusedLdsVec;
constexpr int T_RATIO = P_SAMPLE_MASK, T_RATIO_CL = P_SAMPLE_MASK + 1, T_SELECTED = P_SAMPLE_MASK + 2, T_COUNT = 20;
static_assert(P_SAMPLE_MASK + 3 <= T_COUNT, "token term record too small");

struct FusedArgs {
    nrl_grpo_cfg cfg;
    nrl_grpo_inputs in;  // lp / lpu unused
    const void* logits;
    int64_t n_inner, d_n_inner, vocab, stride_outer, stride_inner;
    const int64_t* targets;
    int64_t ts_outer, ts_inner, vstart, vend;
    float tparam, loss_scale;
    void* dlogits;
    int64_t ds_outer, ds_inner;
    float* lp_out;     // [B, n_inner]
    float* seq_stats;  // [B, 3]: seq_den, seq_w, seq_keep
    float* terms;      // [B * n_inner, T_COUNT]
    double* parts;     // [B, P_COUNT]
    // packed mode (cu != NULL): the logits are one row of `total` positions, sequence s occupies
    // [cu[s], cu[s+1]); the loss inputs stay [n_seq, n_inner]
    const int32_t* cu;
    int64_t n_seq;
    int pre_rolled;
    int4* row_pos;     // packed mode: [total] (sequence, position or -1, target index, 0), filled before the pass
};

// where a logits row sits in the loss inputs: sequence o, position i (i >= n_inner: the row feeds no token),
// and the index of its target id
struct FusedPos {
    int64_t o, i, tgt;
};
__device__ __forceinline__ FusedPos fused_where_packed(const FusedArgs& a, int64_t r, int64_t total) {
    FusedPos q;
    const int64_t seq = find_seq(a.cu, a.n_seq, r);
    q.o = seq < 0 ? 0 : seq;
    q.i = -1;
    q.tgt = 0;
    if (seq >= 0) {
        const int64_t start = a.cu[seq], len = a.cu[seq + 1] - start, pos = r - start;
        if (pos + 1 < len && pos < a.n_inner) q.i = pos;  // the last position of a sequence predicts nothing
        q.tgt = start + (a.pre_rolled ? pos : (pos + 1 < len ? pos + 1 : 0));
        // (the targets hold at least `total` entries; boundaries that run past the packed row cannot index beyond them)
        if (q.tgt >= total) q.tgt = total - 1;
    }
    return q;
}
// The search through the boundaries is a chain of dependent loads; done once per row ahead of the pass,
// the persistent kernel finds a row's place with a single load.
__global__ __launch_bounds__(256) void fused_row_pos_kernel(FusedArgs a, int64_t total) {
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= total) return;
    const FusedPos q = fused_where_packed(a, r, total);
    a.row_pos[r] = make_int4(static_cast<int>(q.o), static_cast<int>(q.i), static_cast<int>(q.tgt), 0);
}
template <bool PACKED>
__device__ __forceinline__ FusedPos fused_where(const FusedArgs& a, int64_t r) {
    FusedPos q;
    if (!PACKED) {
        q.o = r / a.d_n_inner;
        q.i = r - q.o * a.d_n_inner;
        q.tgt = q.o * a.ts_outer + q.i * a.ts_inner;
        return q;
    }
    const int4 p = a.row_pos[r];
    q.o = p.x;
    q.i = p.y < 0 ? a.n_inner : p.y;
    q.tgt = p.z;
    return q;
}
template <bool PACKED>
__device__ __forceinline__ int64_t fused_row_offset(const FusedArgs& a, int64_t r, int64_t so, int64_t si) {
    if (PACKED) return r * si;
    const int64_t o = r / a.d_n_inner;
    return o * so + (r - o * a.d_n_inner) * si;
}

__global__ __launch_bounds__(kLossBlock) void grpo_seq_stats_kernel(FusedArgs a) {
    __shared__ double sm_d[kLossWaves];
    const nrl_grpo_cfg& c = a.cfg;
    const nrl_grpo_inputs& in = a.in;
    const int64_t b = blockIdx.x, n = in.sm1;
    const float smv = in.sample_mask[b];
    double s_tm = 0, s_is = 0, s_geo = 0;
    const bool need_prev = c.sequence_level_importance_ratios || c.tis_type == NRL_TIS_SEQ_MASK;
    for (int64_t t = threadIdx.x; t < n; t += kLossBlock) {
        const float tm = in.token_mask[b * in.token_mask_stride + t];
        s_tm += tm;
        if (need_prev) {
            const float d = in.prev[b * in.prev_stride + t] - in.gen[b * in.gen_stride + t];
            s_is += d * (tm * smv);
            s_geo += finite_or_zero(d) * tm;
        }
    }
    const float seq_den = static_cast<float>(block_sum<double, kLossWaves>(s_tm, sm_d)) + 1e-8f;
    float seq_w = 1.f, seq_keep = 1.f;
    if (c.sequence_level_importance_ratios) seq_w = finite_or_zero(expf(static_cast<float>(block_sum<double, kLossWaves>(s_is, sm_d))));
    if (c.tis_type == NRL_TIS_SEQ_MASK) {
        const float geo = expf(static_cast<float>(block_sum<double, kLossWaves>(s_geo, sm_d)) / seq_den);
        seq_keep = (geo >= c.tis_min && geo <= c.tis_max) ? 1.f : 0.f;
    }
    if (threadIdx.x == 0) {
        a.seq_stats[b * 3] = seq_den;
        a.seq_stats[b * 3 + 1] = seq_w;
        a.seq_stats[b * 3 + 2] = seq_keep;
    }
}

// Persistent workgroups: workgroup w walks rows w, w + gridDim.x, ...  While the gradient of one row
// is being stored, the same slots (registers, and the LDS slice through direct global-to-LDS loads) are
// refilled with the next row this workgroup evaluates, and the online (max, sum) of that row is advanced a few
// vectors behind the loads, so reads, writes and the exponentials all overlap and only the
// cross-wave merge and the one-thread loss evaluation sit between two rows.
// Slot order q = 0 .. kFusedVec-1: the LDS slots come first (vector kFusedRegVec + q), then the
// register slots (vector q - kFusedLdsVec).
// NREG is the number of register slots the instantiation carries (the row must fit NREG + kFusedLdsVec
// slots); shorter rows take a smaller instantiation instead of idling through unused slots.
__global__ void fused_fill_zero_kernel(float* p, int64_t n) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        p[i] = 0.f;
}

template <int DT, int TEMP, int NREG, bool PACKED>
__global__ __launch_bounds__(kFusedBlock) void fused_logits_loss_kernel(FusedArgs a, int64_t n_rows) {
    constexpr int EPV = Row<DT>::EPV;
    constexpr int kFusedRegVec = NREG, kFusedVec = NREG + kFusedLdsVec;
    constexpr int kFusedLag = NREG / 2 < 6 ? NREG / 2 : 6;  // slots between issuing a load and folding it into the running sum
    __shared__ u32x4 stash[kFusedLdsVec * kFusedBlock];
    __shared__ Lse sm_l[kFusedWaves];
    __shared__ float sh_g, sh_lse;
    const nrl_grpo_cfg& c = a.cfg;
    const nrl_grpo_inputs& in = a.in;
    const int tid = threadIdx.x;
    const int nvec = static_cast<int>(a.vocab / EPV);
    const int64_t step = gridDim.x;
    const u32x4 zero = {0u, 0u, 0u, 0u};

    auto out_row = [&](int64_t r) -> char* {
        return static_cast<char*>(a.dlogits) + fused_row_offset<PACKED>(a, r, a.ds_outer, a.ds_inner) * Row<DT>::BYTES;
    };
    auto in_row = [&](int64_t r) -> const char* {
        return static_cast<const char*>(a.logits) + fused_row_offset<PACKED>(a, r, a.stride_outer, a.stride_inner) * Row<DT>::BYTES;
    };
    // Slot q holds vector slot_vec(q) of the row.  Lanes past the end of the row are pointed at the
    // row's last vector instead: they load, compute and store exactly what that vector's own lane does
    // (harmless duplicates), so the slot loop has no divergent branch around its memory operations and
    // the loads of the next row stay in flight behind the stores.
    auto slot_vec = [&](int q) -> int { return tid + (q < kFusedLdsVec ? kFusedRegVec + q : q - kFusedLdsVec) * kFusedBlock; };
    // (recomputed at every use from an opaque copy of the lane index: twenty precomputed offsets would
    // not fit in the register file next to the row)
    auto slot_cl = [&](int q) -> int {
        int t = tid;
        asm volatile("" : "+v"(t));
        return min(t + (q < kFusedLdsVec ? kFusedRegVec + q : q - kFusedLdsVec) * kFusedBlock, nvec - 1);
    };
    auto vec_at = [&](const char* base, int vc) -> const u32x4* {  // uniform base + 32-bit lane offset
        return reinterpret_cast<const u32x4*>(base + static_cast<uint32_t>(vc) * 16u);
    };
    // First row at or after r (in this workgroup's walk) whose token takes part in the loss.  Rows passed
    // over are dropped positions or masked tokens: zero gradient, logprob reported as 0, nothing read.
    auto advance = [&](int64_t r) -> int64_t {
        for (; r < n_rows; r += step) {
            const FusedPos q = fused_where<PACKED>(a, r);
            const int64_t o = q.o, i = q.i;
            float w = 0.f;
            if (i < a.n_inner) w = in.token_mask[o * in.token_mask_stride + i] * in.sample_mask[o];
            if (w != 0.f) break;
            u32x4* ov = reinterpret_cast<u32x4*>(out_row(r));
            for (int v = tid; v < nvec; v += kFusedBlock) ov[v] = zero;
            if (i < a.n_inner) {
                const int64_t tok = o * a.n_inner + i;
                if (tid < T_COUNT) a.terms[tok * T_COUNT + tid] = 0.f;
                if (tid == 0) a.lp_out[tok] = 0.f;
            }
        }
        return r;
    };
    u32x4 regs[kFusedRegVec];
    Lse acc;
    // LDS slot q of the incoming row: global memory -> LDS without passing through registers; each wave
    // fills the 1 KiB of the slot that its own lanes read back
    auto lds_fill = [&](const char* base, int q) {
        u32x4* dst = stash + q * kFusedBlock + (tid & ~(kWave - 1));
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const __attribute__((address_space(1))) void*>(
                                             reinterpret_cast<uintptr_t>(vec_at(base, slot_cl(q)))),
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };
    auto fold = [&](int q) {  // slot q of the incoming row -> running sum; lanes past the row add nothing
        u32x4 raw = q < kFusedLdsVec ? stash[(q < kFusedLdsVec ? q : 0) * kFusedBlock + tid] : regs[q < kFusedLdsVec ? 0 : q - kFusedLdsVec];
        if (slot_vec(q) >= nvec) raw = u32x4{Row<DT>::NEG_INF_WORD, Row<DT>::NEG_INF_WORD, Row<DT>::NEG_INF_WORD, Row<DT>::NEG_INF_WORD};
        float t[EPV];
        Row<DT>::decode(raw, t);
#pragma unroll
        for (int k = 0; k < EPV; ++k) t[k] = scale_logit<DT, TEMP>(t[k], a.tparam);
        lse_push<EPV>(acc, t);
    };
    // the direct-to-LDS loads are not tracked against later LDS reads by the compiler: wait for them
    // (and everything older) by hand before the first read of a refilled LDS slot
    auto wait_lds_fill = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

    int64_t r = advance(blockIdx.x);
    if (r < n_rows) {
        const char* xv = in_row(r);
#pragma unroll
        for (int q = 0; q < kFusedLdsVec; ++q) lds_fill(xv, q);
#pragma unroll
        for (int q = kFusedLdsVec; q < kFusedVec; ++q) regs[q - kFusedLdsVec] = __builtin_nontemporal_load(vec_at(xv, slot_cl(q)));
        acc.m = -FLT_MAX;
        acc.s = 0.f;
#pragma unroll
        for (int q = kFusedLdsVec; q < kFusedVec; ++q) fold(q);
        wait_lds_fill();
#pragma unroll
        for (int q = 0; q < kFusedLdsVec; ++q) fold(q);
    }
    while (r < n_rows) {
        const FusedPos where = fused_where<PACKED>(a, r);
        const int64_t o = where.o, i = where.i;
        const int64_t tok = o * a.n_inner + i;
        const char* row = in_row(r);
        char* ov = out_row(r);
        const Lse tot = block_lse<kFusedWaves>(acc, sm_l);
        const int64_t tg = a.targets[where.tgt];
        const int64_t tloc = (tg >= a.vstart && tg < a.vend) ? tg - a.vstart : -1;
        if (tid == 0) {
            const float log_s = logf(tot.s);
            float lp = 0.f;
            if (tloc >= 0) lp = (scale_logit<DT, TEMP>(Row<DT>::load1(row, tloc), a.tparam) - tot.m) - log_s;
            SeqStats st;
            st.seq_den = a.seq_stats[o * 3]; st.seq_ratio = 1.f; st.seq_w = a.seq_stats[o * 3 + 1]; st.seq_keep = a.seq_stats[o * 3 + 2];
            TokenIn ti;
            ti.lp = lp; ti.lpu = lp;
            ti.prev = c.force_on_policy_ratio ? lp : in.prev[o * in.prev_stride + i];
            ti.gen = in.gen[o * in.gen_stride + i];
            ti.ref = c.has_kl ? in.ref[o * in.ref_stride + i] : 0.f;
            ti.adv = in.adv[o * in.adv_stride + i];
            ti.tm = in.token_mask[o * in.token_mask_stride + i];
            ti.smv = in.sample_mask[o];
            ti.correct = 0.f;
            ti.den_s = in.global_valid[0] + 1e-8f;
            ti.den_t = in.global_valid[1] + 1e-8f;
            const TokenOut out = token_eval<false>(c, st, ti);
            float* rec = a.terms + tok * T_COUNT;
#pragma unroll
            for (int k = 0; k < P_SAMPLE_MASK; ++k) rec[k] = out.term[k];
            rec[T_RATIO] = out.ratio;
            rec[T_RATIO_CL] = out.ratio_cl;
            rec[T_SELECTED] = out.selected ? 1.f : 0.f;
            a.lp_out[tok] = lp;
            sh_g = (out.d_actor + out.d_lpu) * a.loss_scale;
            sh_lse = tot.m + log_s;
        }
        __syncthreads();
        const float g = sh_g, lse = sh_lse;
        const int64_t rn = advance(r + step);
        const char* nx = rn < n_rows ? in_row(rn) : row;
        const int tvec = tloc >= 0 ? static_cast<int>(tloc / EPV) : -1;
        const int tsub = tloc >= 0 ? static_cast<int>(tloc % EPV) : -1;
        const RowGrad rg(lse, g, a.tparam);
        acc.m = -FLT_MAX;
        acc.s = 0.f;
        // The LDS slots first: once all of them are consumed they are refilled for the next row (after
        // the last row the refills and loads re-read the current row and are ignored).
#pragma unroll
        for (int q = 0; q < kFusedLdsVec; ++q) {
            const int vc = slot_cl(q);
            const u32x4 d = grad_vec<DT, TEMP>(stash[q * kFusedBlock + tid], vc == tvec ? tsub : -1, rg);
            __builtin_nontemporal_store(d, const_cast<u32x4*>(vec_at(ov, vc)));
        }
#pragma unroll
        for (int q = 0; q < kFusedLdsVec; ++q) lds_fill(nx, q);
#pragma unroll
        for (int q = kFusedLdsVec; q < kFusedVec; ++q) {
            const int vc = slot_cl(q);
            const u32x4 d = grad_vec<DT, TEMP>(regs[q - kFusedLdsVec], vc == tvec ? tsub : -1, rg);
            __builtin_nontemporal_store(d, const_cast<u32x4*>(vec_at(ov, vc)));
            regs[q - kFusedLdsVec] = __builtin_nontemporal_load(vec_at(nx, vc));
            __builtin_amdgcn_sched_barrier(0);  // keep the fold behind this slot's memory operations ...
            if (q >= kFusedLdsVec + kFusedLag) {
                fold(q - kFusedLag);
                asm volatile("" : "+v"(acc.m), "+v"(acc.s));  // a use right here, so the fold is not sunk past the loop
            }
            __builtin_amdgcn_sched_barrier(0);  // ... and ahead of the next slot's
        }
#pragma unroll
        for (int q = kFusedVec - kFusedLag; q < kFusedVec; ++q) fold(q);
        wait_lds_fill();
#pragma unroll
        for (int q = 0; q < kFusedLdsVec; ++q) fold(q);
        // sh_g / sh_lse are rewritten only after the next block_lse, whose barriers every thread passes
        // after reading them above
        r = rn;
    }
}

// one workgroup per sequence: token term records -> the sequence's row of partials.  Thread t sums the records of
// tokens t, t + 256, ... in that order (the assignment of the three-pass kernel, so both give the same sums); a
// record is read as ten 8-byte pairs, four records in flight per thread (eight measured slower).
__global__ __launch_bounds__(kLossBlock) void grpo_terms_reduce_kernel(FusedArgs a) {
    __shared__ double sm_d[kLossWaves];
    __shared__ float sm_f[kLossWaves];
    static_assert(T_COUNT % 2 == 0, "records are read as 8-byte pairs");
    constexpr int kPairs = T_COUNT / 2, kAhead = 4;
    const int64_t b = blockIdx.x, n = a.n_inner;
    double acc[P_R_MIN];
#pragma unroll
    for (int k = 0; k < P_R_MIN; ++k) acc[k] = 0;
    float r_min = INFINITY, r_max = -INFINITY, rc_min = INFINITY, rc_max = -INFINITY;
    for (int64_t t0 = threadIdx.x; t0 < n; t0 += kAhead * kLossBlock) {
        float2 v[kAhead][kPairs];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const int64_t t = t0 + u * kLossBlock;
            if (t < n) {
                const float2* rec = reinterpret_cast<const float2*>(a.terms + (b * n + t) * T_COUNT);  // 8-byte aligned: T_COUNT is even
#pragma unroll
                for (int k = 0; k < kPairs; ++k) v[u][k] = rec[k];
            }
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            if (t0 + u * kLossBlock >= n) break;
            float rec[T_COUNT];
#pragma unroll
            for (int k = 0; k < kPairs; ++k) { rec[2 * k] = v[u][k].x; rec[2 * k + 1] = v[u][k].y; }
#pragma unroll
            for (int k = 0; k < P_SAMPLE_MASK; ++k) acc[k] += rec[k];
            if (rec[T_SELECTED] != 0.f) {
                r_min = fminf(r_min, rec[T_RATIO]); r_max = fmaxf(r_max, rec[T_RATIO]);
                rc_min = fminf(rc_min, rec[T_RATIO_CL]); rc_max = fmaxf(rc_max, rec[T_RATIO_CL]);
            }
        }
    }
    SeqStats st;
    st.seq_den = a.seq_stats[b * 3]; st.seq_ratio = 1.f; st.seq_w = a.seq_stats[b * 3 + 1]; st.seq_keep = a.seq_stats[b * 3 + 2];
    store_row_parts(a.cfg, a.parts + b * P_COUNT, acc, r_min, r_max, rc_min, rc_max, st, a.in.sample_mask[b], sm_d, sm_f);
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

static int grpo_loss_impl(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float* loss_out, float* dlp_out, float* dlpu_out,
                          float* metrics_out, double* parts, void* stream, const char* what) {
    const bool split = in->lpu != nullptr && cfg->has_kl;
    GrpoArgs a;
    a.cfg = *cfg;
    a.in = *in;
    if (!cfg->has_kl) a.in.lpu = nullptr;
    a.dlp = dlp_out;
    a.dlpu = split ? dlpu_out : nullptr;
    a.parts = parts;
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
    return check_launch(what);
}

// argument checks shared by the two loss entry points (everything except the workspace)
static int grpo_loss_check(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, const float* loss_out, const float* dlp_out,
                           const float* dlpu_out, const float* metrics_out) {
    if (!cfg) return fail(NRL_E_INVALID, "cfg is NULL");
    if (int e = check_inputs(in, !cfg->force_on_policy_ratio, cfg->has_kl != 0, true)) return e;
    if (cfg->kl_type < 1 || cfg->kl_type > 3) return fail(NRL_E_INVALID, "kl_type must be 1, 2 or 3");
    if (cfg->tis_type < 0 || cfg->tis_type > 3) return fail(NRL_E_INVALID, "bad tis_type");
    if (cfg->sequence_level_importance_ratios && cfg->token_level_loss)
        return fail(NRL_E_INVALID, "sequence-level importance ratios need a sequence-level loss");
    if (cfg->has_nll && !in->correct_mask) return fail(NRL_E_INVALID, "correct_mask is NULL");
    if (!loss_out || !metrics_out) return fail(NRL_E_INVALID, "null output");
    const bool split = in->lpu != nullptr && cfg->has_kl;
    if (in->batch * in->sm1 > 0 && (!dlp_out || (split && !dlpu_out))) return fail(NRL_E_INVALID, "null gradient output");
    return NRL_OK;
}

extern "C" int nrl_grpo_loss_fwd_bwd(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float* loss_out, float* dlp_out,
                                     float* dlpu_out, float* metrics_out, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
    if (int e = grpo_loss_check(cfg, in, loss_out, dlp_out, dlpu_out, metrics_out)) return e;
    if (!workspace) return fail(NRL_E_INVALID, "null workspace");
    if (workspace_bytes < nrl_grpo_loss_workspace_bytes(in->batch)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 7) return fail(NRL_E_INVALID, "workspace must be 8-byte aligned");
    return grpo_loss_impl(cfg, in, loss_out, dlp_out, dlpu_out, metrics_out, static_cast<double*>(workspace), stream,
                          "grpo_loss_fwd_bwd");
}

// ---------------------------------------------------------------------------------------------
// The same loss for callers that cannot allocate: the per-sequence partial sums live in a fixed
// device array instead of a caller workspace.  Every GPU holds its own copy of the array at its own
// address; the name `scratch` is only a host-side handle, the address comes from hipGetSymbolAddress
// once per device and is what the kernels receive.
// ---------------------------------------------------------------------------------------------
namespace nrl {
constexpr int64_t kStaticMaxBatch = NRL_GRPO_STATIC_MAX_BATCH;
constexpr int kStaticMaxDevices = 64;
static __device__ __align__(256) double scratch[kStaticMaxBatch * P_COUNT];  // 1.25 MiB per GPU
static std::mutex scratch_mutex;
static double* scratch_ptr[kStaticMaxDevices] = {nullptr};

// device address of this GPU's `scratch`, resolved on the first call with that GPU current
static int scratch_for_current_device(double** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(NRL_E_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kStaticMaxDevices) return fail(NRL_E_UNSUPPORTED, "device index %d beyond %d", dev, kStaticMaxDevices);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(NRL_E_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
        scratch_ptr[dev] = static_cast<double*>(p);
    }
    *out = scratch_ptr[dev];
    return NRL_OK;
}
}  // namespace nrl

extern "C" int nrl_grpo_loss_fwd_bwd_static(const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float* loss_out,
                                            float* dlp_out, float* dlpu_out, float* metrics_out, void* stream) {
    if (int e = grpo_loss_check(cfg, in, loss_out, dlp_out, dlpu_out, metrics_out)) return e;
    if (in->batch > kStaticMaxBatch)
        return fail(NRL_E_WORKSPACE, "batch %lld exceeds the %lld sequences the static scratch holds; use nrl_grpo_loss_fwd_bwd",
                    (long long)in->batch, (long long)kStaticMaxBatch);
    double* parts = nullptr;
    if (int e = scratch_for_current_device(&parts)) return e;
    // rows 0 .. batch-1 of the scratch are rewritten in full by the first launch before the second reads
    // them, and nothing beyond `batch` rows is read, so a previous call's contents need no clearing
    return grpo_loss_impl(cfg, in, loss_out, dlp_out, dlpu_out, metrics_out, parts, stream, "grpo_loss_fwd_bwd_static");
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

// ---------------------------------------------------------------------------------------------
// The two helpers of the loss that the driver also calls on their own (KL in the reward, mean reward):
// calculate_kl element by element, masked_mean row by row.  [B, S]-sized, latency bound.
// ---------------------------------------------------------------------------------------------
struct KlArgs {
    const float* lp;
    const float* ref;
    const float* weight;  // importance sampling weights or NULL
    int64_t n;
    int kl_type, has_in, has_out;
    float in_clamp, out_clamp;
};

struct KlPoint {
    float value, d_logr, d_weight;  // clamped value; d value / d (ref - lp); d value / d weight
};

__device__ __forceinline__ KlPoint kl_point(const KlArgs& a, int64_t i) {
    float logr = a.ref[i] - a.lp[i];
    float in_range = 1.f;
    if (a.has_in) {
        const float cl = clampf(logr, -a.in_clamp, a.in_clamp);
        if (!(logr == cl)) in_range = 0.f;  // a clamped token passes no gradient, neither through the KL nor the weight
        logr = cl;
    }
    const float w = a.weight ? a.weight[i] : 1.f;
    const float k = kl_value(a.kl_type, logr);
    KlPoint o;
    o.value = a.weight ? w * k : k;
    o.d_logr = w * kl_slope(a.kl_type, logr) * in_range;
    o.d_weight = k * in_range;
    if (a.has_out) {
        if (!(o.value >= -a.out_clamp && o.value <= a.out_clamp)) { o.d_logr = 0.f; o.d_weight = 0.f; }
        o.value = clampf(o.value, -a.out_clamp, a.out_clamp);
    }
    return o;
}

__global__ __launch_bounds__(256) void calculate_kl_kernel(KlArgs a, float* out) {
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < a.n; i += gridDim.x * 256ll) out[i] = kl_point(a, i).value;
}

__global__ __launch_bounds__(256) void calculate_kl_bwd_kernel(KlArgs a, const float* g, float* d_lp, float* d_ref, float* d_weight) {
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < a.n; i += gridDim.x * 256ll) {
        const KlPoint p = kl_point(a, i);
        const float t = g[i] * p.d_logr;
        if (d_lp) d_lp[i] = -t;
        if (d_ref) d_ref[i] = t;
        if (d_weight) d_weight[i] = g[i] * p.d_weight;
    }
}

static int kl_args(KlArgs& a, const float* lp, const float* ref, const float* weight, int64_t n, int32_t kl_type,
                   int32_t has_in, float in_clamp, int32_t has_out, float out_clamp) {
    if (n < 0 || (n > 0 && (!lp || !ref))) return fail(NRL_E_INVALID, "calculate_kl: null input");
    if (kl_type < 1 || kl_type > 3) return fail(NRL_E_INVALID, "calculate_kl: kl_type must be 1 (k1), 2 (k2) or 3 (k3)");
    a = KlArgs{lp, ref, weight, n, kl_type, has_in, has_out, in_clamp, out_clamp};
    return NRL_OK;
}

static unsigned small_grid(int64_t n) { return static_cast<unsigned>(n + 255 < 256 * 2048ll ? (n + 255) / 256 : 2048); }

extern "C" int nrl_calculate_kl(const float* logprobs, const float* logprobs_reference, const float* weights, int64_t n,
                                int32_t kl_type, int32_t has_input_clamp, float input_clamp, int32_t has_output_clamp,
                                float output_clamp, float* kl_out, void* stream) {
    KlArgs a;
    if (int e = kl_args(a, logprobs, logprobs_reference, weights, n, kl_type, has_input_clamp, input_clamp,
                        has_output_clamp, output_clamp)) return e;
    if (n == 0) return NRL_OK;
    if (!kl_out) return fail(NRL_E_INVALID, "calculate_kl: null output");
    calculate_kl_kernel<<<dim3(small_grid(n)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(a, kl_out);
    return check_launch("calculate_kl");
}

extern "C" int nrl_calculate_kl_bwd(const float* grad_kl, const float* logprobs, const float* logprobs_reference,
                                    const float* weights, int64_t n, int32_t kl_type, int32_t has_input_clamp,
                                    float input_clamp, int32_t has_output_clamp, float output_clamp, float* dlogprobs_out,
                                    float* dreference_out, float* dweights_out, void* stream) {
    KlArgs a;
    if (int e = kl_args(a, logprobs, logprobs_reference, weights, n, kl_type, has_input_clamp, input_clamp,
                        has_output_clamp, output_clamp)) return e;
    if (n == 0) return NRL_OK;
    if (!grad_kl) return fail(NRL_E_INVALID, "calculate_kl_bwd: null upstream gradient");
    if (dweights_out && !weights) return fail(NRL_E_INVALID, "calculate_kl_bwd: a weight gradient without weights");
    calculate_kl_bwd_kernel<<<dim3(small_grid(n)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        a, grad_kl, dlogprobs_out, dreference_out, dweights_out);
    return check_launch("calculate_kl_bwd");
}

// one workgroup per row: out[r] = sum_c(values * mask) / (norm + 1e-8), norm = sum_c(mask) unless given
__global__ __launch_bounds__(kLossBlock) void masked_mean_kernel(const float* values, const float* mask, int64_t n_cols,
                                                                 const float* norm_dev, float norm_host, int has_norm,
                                                                 float* out, float* denom_out) {
    __shared__ double red[kLossBlock / kWave];
    const int64_t r = blockIdx.x;
    double sv = 0.0, sm = 0.0;
    for (int64_t c = threadIdx.x; c < n_cols; c += kLossBlock) {
        const float m = mask[r * n_cols + c];
        sv += static_cast<double>(values[r * n_cols + c] * m);
        sm += static_cast<double>(m);
    }
    sv = block_sum<double, kLossBlock / kWave>(sv, red);
    __syncthreads();
    sm = block_sum<double, kLossBlock / kWave>(sm, red);
    if (threadIdx.x == 0) {
        const float norm = has_norm ? (norm_dev ? norm_dev[0] : norm_host) : static_cast<float>(sm);
        const float den = norm + 1e-8f;
        out[r] = static_cast<float>(sv) / den;
        if (denom_out) denom_out[r] = den;
    }
}

__global__ __launch_bounds__(256) void masked_mean_bwd_kernel(const float* g, const float* mask, const float* denom,
                                                              int64_t n_rows, int64_t n_cols, float* d_values) {
    const int64_t n = n_rows * n_cols;
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += gridDim.x * 256ll) {
        const int64_t r = i / n_cols;
        d_values[i] = g[r] * mask[i] / denom[r];
    }
}

extern "C" int nrl_masked_mean(const float* values, const float* mask, int64_t n_rows, int64_t n_cols,
                               const float* norm_device, float norm_host, int32_t has_norm, float* out, float* denom_out,
                               void* stream) {
    if (n_rows < 0 || n_cols < 0) return fail(NRL_E_INVALID, "masked_mean: negative shape");
    if (n_rows == 0) return NRL_OK;
    if (!out || (n_cols > 0 && (!values || !mask))) return fail(NRL_E_INVALID, "masked_mean: null pointer");
    if (n_rows > 0x7fffffffll) return fail(NRL_E_UNSUPPORTED, "masked_mean: more than 2^31 - 1 rows");
    masked_mean_kernel<<<dim3((unsigned)n_rows), dim3(kLossBlock), 0, static_cast<hipStream_t>(stream)>>>(
        values, mask, n_cols, norm_device, norm_host, has_norm, out, denom_out);
    return check_launch("masked_mean");
}

extern "C" int nrl_masked_mean_bwd(const float* grad_out, const float* mask, const float* denom, int64_t n_rows,
                                   int64_t n_cols, float* dvalues_out, void* stream) {
    if (n_rows < 0 || n_cols < 0) return fail(NRL_E_INVALID, "masked_mean_bwd: negative shape");
    if (n_rows * n_cols == 0) return NRL_OK;
    if (!grad_out || !mask || !denom || !dvalues_out) return fail(NRL_E_INVALID, "masked_mean_bwd: null pointer");
    masked_mean_bwd_kernel<<<dim3(small_grid(n_rows * n_cols)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        grad_out, mask, denom, n_rows, n_cols, dvalues_out);
    return check_launch("masked_mean_bwd");
}

static int64_t align8(int64_t v) { return (v + 7) / 8 * 8; }

extern "C" int64_t nrl_fused_workspace_bytes(int64_t batch, int64_t n_inner) {
    const int64_t b = batch < 1 ? 1 : batch, n = n_inner < 1 ? 1 : n_inner;
    return align8(b * 3 * 4) + align8(b * n * T_COUNT * 4) + b * P_COUNT * 8;
}

extern "C" int64_t nrl_fused_packed_workspace_bytes(int64_t n_seq, int64_t n_inner, int64_t total) {
    return nrl_fused_workspace_bytes(n_seq, n_inner) + 16 + (total < 1 ? 1 : total) * 16;
}

// rows describes the logits; with cu != NULL it is one packed row of rows->n_inner positions (n_outer 1) and
// the loss inputs are [n_seq, in->sm1]
static int fused_impl(const nrl_rows* rows, const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in, float loss_scale, void* dlogits,
                      int64_t d_n_inner, int64_t d_stride_outer, int64_t d_stride_inner, float* logprob_out, float* loss_out,
                      float* metrics_out, void* workspace, int64_t workspace_bytes, void* stream, const int32_t* cu,
                      int64_t n_seq, int pre_rolled) {
    if (!rows || !cfg || !in) return fail(NRL_E_INVALID, "null argument");
    if (rows->dtype != NRL_F32 && rows->dtype != NRL_BF16 && rows->dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown logits dtype");
    if (rows->n_outer < 0 || rows->n_inner < 0 || rows->vocab <= 0 || d_n_inner < rows->n_inner) return fail(NRL_E_INVALID, "bad shape");
    if (!cu && (in->batch != rows->n_outer || in->sm1 != rows->n_inner)) return fail(NRL_E_INVALID, "loss inputs and logits rows disagree");
    if (cu && (in->batch != n_seq || rows->n_outer != 1 || n_seq < 0)) return fail(NRL_E_INVALID, "packed loss inputs and cu_seqlens disagree");
    if (rows->vocab_end - rows->vocab_start != rows->vocab) return fail(NRL_E_INVALID, "vocab range does not span the columns");
    if (!(rows->temperature > 0.f)) return fail(NRL_E_INVALID, "temperature must be positive");
    const bool gspo = cfg->sequence_level_importance_ratios && !cfg->disable_ppo_ratio && !cfg->force_on_policy_ratio;
    if (gspo) return fail(NRL_E_UNSUPPORTED, "sequence-level probability ratios need every logprob of a sequence first");
    if (cfg->has_nll) return fail(NRL_E_UNSUPPORTED, "the positive-example NLL term is not fused");
    // sequence-level importance weights are sums over prev - gen; with force_on_policy_ratio prev is the
    // current logprob itself, which does not exist before the pass
    const bool seq_weights = cfg->sequence_level_importance_ratios || cfg->tis_type == NRL_TIS_SEQ_MASK;
    if (seq_weights && cfg->force_on_policy_ratio)
        return fail(NRL_E_UNSUPPORTED, "sequence-level importance weights with force_on_policy_ratio depend on the current logprobs");
    if (seq_weights && in->batch * in->sm1 > 0 && !in->prev) return fail(NRL_E_INVALID, "prev_logprobs is NULL");
    if (cfg->kl_type < 1 || cfg->kl_type > 3 || cfg->tis_type < 0 || cfg->tis_type > 3) return fail(NRL_E_INVALID, "bad kl_type or tis_type");
    const int bytes = rows->dtype == NRL_F32 ? 4 : 2, epv = 16 / bytes;
    if (rows->vocab % epv || rows->vocab / epv > static_cast<int64_t>(kFusedMaxVec) * kFusedBlock)
        return fail(NRL_E_UNSUPPORTED, "row does not fit the on-chip path (vocab %lld)", (long long)rows->vocab);
    if ((reinterpret_cast<uintptr_t>(rows->logits) & 15) || (reinterpret_cast<uintptr_t>(dlogits) & 15) ||
        (rows->stride_outer * bytes) % 16 || (rows->stride_inner * bytes) % 16 || (d_stride_outer * bytes) % 16 ||
        (d_stride_inner * bytes) % 16)
        return fail(NRL_E_UNSUPPORTED, "rows must be 16-byte aligned");
    const int64_t n_rows = rows->n_outer * d_n_inner;
    if (n_rows >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    if (!loss_out || !metrics_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    const int64_t need = cu ? nrl_fused_packed_workspace_bytes(in->batch, in->sm1, n_rows) : nrl_fused_workspace_bytes(in->batch, in->sm1);
    if (workspace_bytes < need) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 7) return fail(NRL_E_INVALID, "workspace must be 8-byte aligned");
    if (n_rows > 0) {
        if (!rows->logits || !rows->targets || !dlogits || !logprob_out) return fail(NRL_E_INVALID, "null logits, targets or output");
        if (!in->gen || !in->adv || !in->token_mask || !in->sample_mask || !in->global_valid) return fail(NRL_E_INVALID, "null loss input");
        if (!cfg->force_on_policy_ratio && !in->prev) return fail(NRL_E_INVALID, "prev_logprobs is NULL");
        if (cfg->has_kl && !in->ref) return fail(NRL_E_INVALID, "reference_policy_logprobs is NULL");
    }
    FusedArgs a;
    a.cfg = *cfg;
    a.in = *in;
    a.in.lp = nullptr; a.in.lpu = nullptr;
    a.cu = cu; a.n_seq = n_seq; a.pre_rolled = pre_rolled;
    a.logits = rows->logits; a.n_inner = in->sm1; a.d_n_inner = d_n_inner; a.vocab = rows->vocab;
    a.stride_outer = rows->stride_outer; a.stride_inner = rows->stride_inner;
    a.targets = rows->targets; a.ts_outer = rows->tgt_stride_outer; a.ts_inner = rows->tgt_stride_inner;
    a.vstart = rows->vocab_start; a.vend = rows->vocab_end;
    a.loss_scale = loss_scale;
    a.dlogits = dlogits; a.ds_outer = d_stride_outer; a.ds_inner = d_stride_inner;
    a.lp_out = logprob_out;
    char* ws = static_cast<char*>(workspace);
    a.seq_stats = reinterpret_cast<float*>(ws); ws += align8(in->batch * 3 * 4);
    a.terms = reinterpret_cast<float*>(ws); ws += align8(in->batch * (in->sm1 < 1 ? 1 : in->sm1) * T_COUNT * 4);
    a.parts = reinterpret_cast<double*>(ws); ws += in->batch * P_COUNT * 8;
    a.row_pos = cu ? reinterpret_cast<int4*>(ws + ((16 - (reinterpret_cast<uintptr_t>(ws) & 15)) & 15)) : nullptr;
    int tc = 0;
    a.tparam = 1.f;
    if (rows->temperature != 1.0f) {
        if (rows->temp_mode == NRL_TEMP_DIV) { tc = 1; a.tparam = rows->temperature; }
        else { tc = 2; a.tparam = 1.0f / rows->temperature; }
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const unsigned nb = static_cast<unsigned>(in->batch);
    if (nb > 0) grpo_seq_stats_kernel<<<dim3(nb), dim3(kLossBlock), 0, s>>>(a);
    if (cu && in->batch * in->sm1 > 0) {
        // positions past a sequence's end have no packed row: their records and logprobs start at zero
        fused_fill_zero_kernel<<<dim3(1024), dim3(256), 0, s>>>(a.terms, in->batch * in->sm1 * T_COUNT);
        fused_fill_zero_kernel<<<dim3(256), dim3(256), 0, s>>>(a.lp_out, in->batch * in->sm1);
    }
    if (cu && n_rows > 0) fused_row_pos_kernel<<<dim3((unsigned)((n_rows + 255) / 256)), dim3(256), 0, s>>>(a, n_rows);
    if (n_rows > 0) {
        int dev = 0, cus = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1)
            return fail(NRL_E_LAUNCH, "cannot read the device's compute-unit count");
        // one resident workgroup per compute unit (64 KiB of LDS and 1024 threads each)
        const dim3 grid((unsigned)(n_rows < cus ? n_rows : cus)), block(kFusedBlock);
        const int64_t slots = (rows->vocab / epv + kFusedBlock - 1) / kFusedBlock;
        const int nreg = slots <= 8 ? 4 : slots <= 12 ? 8 : slots <= 16 ? 12 : 16;
#define NRL_FUSED_LAUNCH(DT_, TC_, NR_)                                                                           \
    if (cu) fused_logits_loss_kernel<DT_, TC_, NR_, true><<<grid, block, 0, s>>>(a, n_rows);                      \
    else fused_logits_loss_kernel<DT_, TC_, NR_, false><<<grid, block, 0, s>>>(a, n_rows)
#define NRL_FUSED_CASE(DT_, TC_)                                                                                  \
    case DT_ * 3 + TC_:                                                                                           \
        if (nreg == 4) { NRL_FUSED_LAUNCH(DT_, TC_, 4); }                                                         \
        else if (nreg == 8) { NRL_FUSED_LAUNCH(DT_, TC_, 8); }                                                    \
        else if (nreg == 12) { NRL_FUSED_LAUNCH(DT_, TC_, 12); }                                                  \
        else { NRL_FUSED_LAUNCH(DT_, TC_, 16); }                                                                  \
        break;
        switch (rows->dtype * 3 + tc) {
            NRL_FUSED_CASE(NRL_F32, 0) NRL_FUSED_CASE(NRL_F32, 1) NRL_FUSED_CASE(NRL_F32, 2)
            NRL_FUSED_CASE(NRL_BF16, 0) NRL_FUSED_CASE(NRL_BF16, 1) NRL_FUSED_CASE(NRL_BF16, 2)
            NRL_FUSED_CASE(NRL_F16, 0) NRL_FUSED_CASE(NRL_F16, 1) NRL_FUSED_CASE(NRL_F16, 2)
            default: return fail(NRL_E_INVALID, "unknown logits dtype");
        }
#undef NRL_FUSED_CASE
#undef NRL_FUSED_LAUNCH
    }
    if (nb > 0) grpo_terms_reduce_kernel<<<dim3(nb), dim3(kLossBlock), 0, s>>>(a);
    GrpoArgs fa;
    fa.cfg = *cfg;
    fa.in = *in;
    fa.dlp = nullptr; fa.dlpu = nullptr;
    fa.parts = a.parts;
    grpo_finish_kernel<<<dim3(1), dim3(kLossBlock), 0, s>>>(fa, loss_out, metrics_out);
    return check_launch("fused_logits_grpo_loss");
}

extern "C" int nrl_fused_logits_grpo_loss(const nrl_rows* rows, const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in,
                                          float loss_scale, void* dlogits, int64_t d_n_inner, int64_t d_stride_outer,
                                          int64_t d_stride_inner, float* logprob_out, float* loss_out, float* metrics_out,
                                          void* workspace, int64_t workspace_bytes, void* stream) {
    return fused_impl(rows, cfg, in, loss_scale, dlogits, d_n_inner, d_stride_outer, d_stride_inner, logprob_out, loss_out,
                      metrics_out, workspace, workspace_bytes, stream, nullptr, 0, 0);
}

extern "C" int nrl_fused_packed_logits_grpo_loss(const nrl_rows* rows, int32_t target_is_pre_rolled, const int32_t* cu_seqlens,
                                                 int64_t n_seq, const nrl_grpo_cfg* cfg, const nrl_grpo_inputs* in,
                                                 float loss_scale, void* dlogits, int64_t d_row_stride, float* logprob_out,
                                                 float* loss_out, float* metrics_out, void* workspace, int64_t workspace_bytes,
                                                 void* stream) {
    if (!cu_seqlens) return fail(NRL_E_INVALID, "cu_seqlens is NULL");
    if (rows && rows->tgt_stride_inner != 1) return fail(NRL_E_INVALID, "packed targets must be contiguous");
    return fused_impl(rows, cfg, in, loss_scale, dlogits, rows ? rows->n_inner : 0, 0, d_row_stride, logprob_out, loss_out,
                      metrics_out, workspace, workspace_bytes, stream, cu_seqlens, n_seq, target_is_pre_rolled);
}

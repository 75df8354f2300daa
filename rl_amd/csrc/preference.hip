// Preference losses on token logprobs: DPO (rewards = masked sums of logprob - reference logprob per
// sequence, pairs of chosen / rejected rows), the plain reward-model preference loss, and the
// per-sample NLL rows that DPO's SFT term is built from.  All of it is [B, S] work: one workgroup per
// sequence for the row sums (fp64 accumulation), one workgroup over the pairs for the scalar terms
// (fixed order, so the result does not depend on the launch), one elementwise launch for the gradient.

#include <float.h>
#include <math.h>

#include "common.hpp"

namespace nrl {

constexpr int kPrefBlock = 256;
constexpr int kPrefWaves = kPrefBlock / kWave;

struct PrefArgs {
    const float* lp;           // [B, n]
    const float* ref;          // [B, n] or NULL (zeros)
    const float* token_mask;   // [B, n]
    const float* sample_mask;  // [B]
    const float* global_valid; // [0] = valid sequences over the global batch
    const float* rewards;      // [B]: given rewards (reward-model loss) or the row kernel's output
    int64_t batch, n, lp_stride, ref_stride, tm_stride;
    float beta, w_pref, w_sft;
    int avg_pref, avg_sft, has_sft;
    float* row;      // [B, 4]: reward, d reward / d logprob, SFT row loss, d SFT row loss / d logprob
    float* coef;     // [B]: d loss / d logprob of an unmasked token of the row (d loss / d reward without rows)
    float* dlp;      // [B, n]
    float* loss;
    float* metrics;  // DPO: 7, reward model: 5
};

__global__ __launch_bounds__(kPrefBlock) void pref_rows_kernel(PrefArgs a) {
    __shared__ double sm[kPrefWaves];
    const int64_t b = blockIdx.x;
    const float smv = a.sample_mask[b];
    double s_tm = 0, s_rew = 0, s_nll = 0, s_nm = 0;
    for (int64_t t = threadIdx.x; t < a.n; t += kPrefBlock) {
        const float tm = a.token_mask[b * a.tm_stride + t];
        const float lp = a.lp[b * a.lp_stride + t];
        const float rf = a.ref ? a.ref[b * a.ref_stride + t] : 0.f;
        s_tm += tm;
        s_rew += static_cast<double>((lp - rf) * tm);
        const float m = tm * smv;
        s_nll += static_cast<double>(lp * m);
        s_nm += m;
    }
    s_tm = block_sum<double, kPrefWaves>(s_tm, sm);
    s_rew = block_sum<double, kPrefWaves>(s_rew, sm);
    s_nll = block_sum<double, kPrefWaves>(s_nll, sm);
    s_nm = block_sum<double, kPrefWaves>(s_nm, sm);
    if (threadIdx.x == 0) {
        const float fp = a.avg_pref ? 1.f / fmaxf(static_cast<float>(s_tm), 1.f) : 1.f;
        const float fs = a.avg_sft ? 1.f / fmaxf(static_cast<float>(s_nm), 1.f) : 1.f;
        float* r = a.row + b * 4;
        r[0] = static_cast<float>(s_rew) * fp;
        r[1] = fp;
        r[2] = -static_cast<float>(s_nll) * fs;
        r[3] = -smv * fs;
    }
}

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// One workgroup: the pairs in ascending order.  ROWS: rewards come from pref_rows_kernel (stride 4) and the
// SFT term may be present; otherwise they are the caller's [B] and beta = 1.
template <bool ROWS>
__global__ __launch_bounds__(kPrefBlock) void pref_finish_kernel(PrefArgs a) {
    __shared__ double sm[kPrefWaves];
    const int64_t pairs = a.batch / 2;
    const float den = a.global_valid[0] / 2.f + 1e-8f;
    const int64_t rs = ROWS ? 4 : 1;
    const float* rew = ROWS ? a.row : a.rewards;
    double s_pref = 0, s_acc = 0, s_rc = 0, s_rr = 0, s_sft = 0, s_sm = 0;
    for (int64_t p = threadIdx.x; p < pairs; p += kPrefBlock) {
        const int64_t c = 2 * p, r = c + 1;
        const float wc = a.sample_mask[c], wr = a.sample_mask[r];
        const float rc = rew[c * rs], rr = rew[r * rs];
        const float x = a.beta * (rc - rr);
        s_pref += static_cast<double>((-log_sigmoid(x) * wc) * wc);
        s_acc += rc > rr ? wc : 0.f;
        s_rc += static_cast<double>(rc * wc);
        s_rr += static_cast<double>(rr * wr);
        s_sm += static_cast<double>(wc) + wr;
        // d(-logsigmoid(x)) / dx = -sigmoid(-x)
        const float g = a.w_pref * (wc * wc / den) * (-a.beta / (1.f + expf(x)));
        float cc = g, cr = -g;
        if (ROWS) {
            cc *= a.row[c * 4 + 1];
            cr *= a.row[r * 4 + 1];
            if (a.has_sft) {
                s_sft += static_cast<double>(a.row[c * 4 + 2] * wc);
                cc += a.w_sft * (wc / den) * a.row[c * 4 + 3];
            }
        }
        a.coef[c] = cc;
        a.coef[r] = cr;
    }
    s_pref = block_sum<double, kPrefWaves>(s_pref, sm);
    s_acc = block_sum<double, kPrefWaves>(s_acc, sm);
    s_rc = block_sum<double, kPrefWaves>(s_rc, sm);
    s_rr = block_sum<double, kPrefWaves>(s_rr, sm);
    s_sft = block_sum<double, kPrefWaves>(s_sft, sm);
    s_sm = block_sum<double, kPrefWaves>(s_sm, sm);
    if (threadIdx.x == 0) {
        const float pref = static_cast<float>(s_pref) / den;
        const float sft = (ROWS && a.has_sft) ? static_cast<float>(s_sft) / den : 0.f;
        const float loss = ROWS ? a.w_sft * sft + a.w_pref * pref : pref;
        *a.loss = loss;
        float* m = a.metrics;
        int k = 0;
        m[k++] = loss;
        if (ROWS) { m[k++] = sft; m[k++] = pref; }
        m[k++] = static_cast<float>(s_acc) / den;
        m[k++] = static_cast<float>(s_rc) / den;
        m[k++] = static_cast<float>(s_rr) / den;
        m[k++] = static_cast<float>(s_sm) / 2.f;
    }
}

__global__ __launch_bounds__(kPrefBlock) void pref_grad_kernel(PrefArgs a) {
    const int64_t total = a.batch * a.n;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kPrefBlock + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * kPrefBlock) {
        const int64_t b = i / a.n, t = i - b * a.n;
        a.dlp[i] = a.token_mask[b * a.tm_stride + t] * a.coef[b];
    }
}

// per-sample NLL: loss[b] = -sum_t lp * tm * sm[b] (/ max(sum_t tm * sm[b], 1)); den[b] is that divisor
__global__ __launch_bounds__(kPrefBlock) void nll_rows_kernel(const float* lp, int64_t lp_stride, const float* tm, int64_t tm_stride,
                                                              const float* sample_mask, int64_t n, int average, float* loss,
                                                              float* den, float* n_unmasked) {
    __shared__ double sm[kPrefWaves];
    const int64_t b = blockIdx.x;
    const float smv = sample_mask[b];
    double s_nll = 0, s_nm = 0;
    for (int64_t t = threadIdx.x; t < n; t += kPrefBlock) {
        const float m = tm[b * tm_stride + t] * smv;
        s_nll += static_cast<double>(lp[b * lp_stride + t] * m);
        s_nm += m;
    }
    s_nll = block_sum<double, kPrefWaves>(s_nll, sm);
    s_nm = block_sum<double, kPrefWaves>(s_nm, sm);
    if (threadIdx.x == 0) {
        const float d = average ? fmaxf(static_cast<float>(s_nm), 1.f) : 1.f;
        loss[b] = -static_cast<float>(s_nll) / d;
        den[b] = d;
        n_unmasked[b] = static_cast<float>(s_nm);
    }
}

__global__ __launch_bounds__(kPrefBlock) void nll_rows_totals_kernel(const float* n_unmasked, const float* sample_mask, int64_t batch,
                                                                     float* totals) {
    __shared__ double sm[kPrefWaves];
    double s_tok = 0, s_sm = 0;
    for (int64_t b = threadIdx.x; b < batch; b += kPrefBlock) { s_tok += n_unmasked[b]; s_sm += sample_mask[b]; }
    s_tok = block_sum<double, kPrefWaves>(s_tok, sm);
    s_sm = block_sum<double, kPrefWaves>(s_sm, sm);
    if (threadIdx.x == 0) { totals[0] = static_cast<float>(s_tok); totals[1] = static_cast<float>(s_sm); }
}

__global__ __launch_bounds__(kPrefBlock) void nll_rows_grad_kernel(const float* grad_rows, const float* tm, int64_t tm_stride,
                                                                   const float* sample_mask, const float* den, int64_t batch,
                                                                   int64_t n, float* dlp) {
    const int64_t total = batch * n;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kPrefBlock + threadIdx.x; i < total; i += static_cast<int64_t>(gridDim.x) * kPrefBlock) {
        const int64_t b = i / n, t = i - b * n;
        dlp[i] = -(tm[b * tm_stride + t] * sample_mask[b]) / den[b] * grad_rows[b];
    }
}

static unsigned grid_for(int64_t total) {
    const int64_t blocks = (total + kPrefBlock - 1) / kPrefBlock;
    return static_cast<unsigned>(blocks < 1 ? 1 : blocks > 4096 ? 4096 : blocks);
}

}  // namespace nrl

using namespace nrl;

extern "C" int64_t nrl_dpo_workspace_bytes(int64_t batch) { return (batch < 1 ? 1 : batch) * 5 * static_cast<int64_t>(sizeof(float)); }

extern "C" int nrl_dpo_loss_fwd_bwd(const float* lp, int64_t lp_stride, const float* ref, int64_t ref_stride,
                                    const float* token_mask, int64_t token_mask_stride, const float* sample_mask,
                                    const float* global_valid, int64_t batch, int64_t n, float beta,
                                    float preference_loss_weight, float sft_loss_weight,
                                    int32_t preference_average_log_probs, int32_t sft_average_log_probs, float* loss_out,
                                    float* dlp_out, float* metrics_out, void* workspace, int64_t workspace_bytes,
                                    void* stream) {
    if (batch < 0 || n < 0) return fail(NRL_E_INVALID, "bad shape [%lld, %lld]", (long long)batch, (long long)n);
    if (batch % 2) return fail(NRL_E_INVALID, "rows come in (chosen, rejected) pairs; got %lld rows", (long long)batch);
    if (batch >= (1ll << 31)) return fail(NRL_E_INVALID, "too many sequences");
    if (!sample_mask && batch > 0) return fail(NRL_E_INVALID, "sample_mask is NULL");
    if (!global_valid || !loss_out || !metrics_out || !workspace) return fail(NRL_E_INVALID, "null argument");
    if (batch * n > 0 && (!lp || !token_mask || !dlp_out)) return fail(NRL_E_INVALID, "null logprobs, token_mask or gradient output");
    if (workspace_bytes < nrl_dpo_workspace_bytes(batch)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 3) return fail(NRL_E_INVALID, "workspace must be 4-byte aligned");
    PrefArgs a;
    a.lp = lp; a.ref = ref; a.token_mask = token_mask; a.sample_mask = sample_mask; a.global_valid = global_valid; a.rewards = nullptr;
    a.batch = batch; a.n = n; a.lp_stride = lp_stride; a.ref_stride = ref_stride; a.tm_stride = token_mask_stride;
    a.beta = beta; a.w_pref = preference_loss_weight; a.w_sft = sft_loss_weight;
    a.avg_pref = preference_average_log_probs; a.avg_sft = sft_average_log_probs; a.has_sft = sft_loss_weight > 0.f;
    a.row = static_cast<float*>(workspace);
    a.coef = a.row + (batch < 1 ? 1 : batch) * 4;
    a.dlp = dlp_out; a.loss = loss_out; a.metrics = metrics_out;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (batch > 0) pref_rows_kernel<<<dim3((unsigned)batch), dim3(kPrefBlock), 0, s>>>(a);
    pref_finish_kernel<true><<<dim3(1), dim3(kPrefBlock), 0, s>>>(a);
    if (batch * n > 0) pref_grad_kernel<<<dim3(grid_for(batch * n)), dim3(kPrefBlock), 0, s>>>(a);
    return check_launch("dpo_loss_fwd_bwd");
}

extern "C" int nrl_preference_loss_fwd_bwd(const float* rewards, const float* sample_mask, const float* global_valid,
                                           int64_t batch, float* loss_out, float* drewards_out, float* metrics_out,
                                           void* stream) {
    if (batch < 0 || batch % 2) return fail(NRL_E_INVALID, "rows come in (chosen, rejected) pairs; got %lld rows", (long long)batch);
    if (batch >= (1ll << 31)) return fail(NRL_E_INVALID, "too many sequences");
    if (!global_valid || !loss_out || !metrics_out) return fail(NRL_E_INVALID, "null argument");
    if (batch > 0 && (!rewards || !sample_mask || !drewards_out)) return fail(NRL_E_INVALID, "null rewards, sample_mask or gradient output");
    PrefArgs a = {};
    a.sample_mask = sample_mask; a.global_valid = global_valid; a.rewards = rewards;
    a.batch = batch; a.beta = 1.f; a.w_pref = 1.f;
    a.coef = drewards_out; a.loss = loss_out; a.metrics = metrics_out;
    pref_finish_kernel<false><<<dim3(1), dim3(kPrefBlock), 0, static_cast<hipStream_t>(stream)>>>(a);
    return check_launch("preference_loss_fwd_bwd");
}

extern "C" int nrl_nll_rows_fwd(const float* lp, int64_t lp_stride, const float* token_mask, int64_t token_mask_stride,
                                const float* sample_mask, int64_t batch, int64_t n, int32_t average_log_probs,
                                float* loss_rows_out, float* den_out, float* totals_out, void* workspace,
                                int64_t workspace_bytes, void* stream) {
    if (batch < 0 || n < 0) return fail(NRL_E_INVALID, "bad shape [%lld, %lld]", (long long)batch, (long long)n);
    if (batch >= (1ll << 31)) return fail(NRL_E_INVALID, "too many sequences");
    if (!totals_out || !workspace) return fail(NRL_E_INVALID, "null argument");
    if (batch > 0 && (!sample_mask || !loss_rows_out || !den_out)) return fail(NRL_E_INVALID, "null sample_mask or output");
    if (batch * n > 0 && (!lp || !token_mask)) return fail(NRL_E_INVALID, "null logprobs or token_mask");
    if (workspace_bytes < (batch < 1 ? 1 : batch) * static_cast<int64_t>(sizeof(float))) return fail(NRL_E_WORKSPACE, "workspace too small");
    hipStream_t s = static_cast<hipStream_t>(stream);
    float* n_unmasked = static_cast<float*>(workspace);
    if (batch > 0)
        nll_rows_kernel<<<dim3((unsigned)batch), dim3(kPrefBlock), 0, s>>>(lp, lp_stride, token_mask, token_mask_stride, sample_mask, n,
                                                                             average_log_probs, loss_rows_out, den_out, n_unmasked);
    nll_rows_totals_kernel<<<dim3(1), dim3(kPrefBlock), 0, s>>>(n_unmasked, sample_mask, batch, totals_out);
    return check_launch("nll_rows_fwd");
}

extern "C" int nrl_nll_rows_bwd(const float* grad_rows, const float* token_mask, int64_t token_mask_stride,
                                const float* sample_mask, const float* den, int64_t batch, int64_t n, float* dlp_out,
                                void* stream) {
    if (batch < 0 || n < 0) return fail(NRL_E_INVALID, "bad shape [%lld, %lld]", (long long)batch, (long long)n);
    if (batch * n == 0) return NRL_OK;
    if (!grad_rows || !token_mask || !sample_mask || !den || !dlp_out) return fail(NRL_E_INVALID, "null argument");
    nll_rows_grad_kernel<<<dim3(grid_for(batch * n)), dim3(kPrefBlock), 0, static_cast<hipStream_t>(stream)>>>(
        grad_rows, token_mask, token_mask_stride, sample_mask, den, batch, n, dlp_out);
    return check_launch("nll_rows_bwd");
}

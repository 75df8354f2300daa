// K5: per-prompt group baseline / std and GRPO advantages.
//
// Rows belong to one group iff their prompt-token rows are exactly equal.  Launch 1 hashes every
// prompt row (one workgroup per row).  Launch 2 finds, for every row, the first row with the same
// content: candidates are pre-filtered by the 64-bit hash and then confirmed with a full
// element-wise comparison, so a hash collision can never merge two different prompts.  Launch 3
// (one thread per row) accumulates the group statistics in ascending row order in fp32 and
// evaluates the reference's formula (E[r^2] - E[r]^2 scaled by n/(n-1), NaN -> 0) unchanged, so
// decisions such as std > 0 come out the same.

#include <float.h>
#include <math.h>

#include "common.hpp"

namespace nrl {

constexpr int kAdvBlock = 256;
constexpr int kAdvWaves = kAdvBlock / kWave;

__device__ __forceinline__ uint64_t mix64(uint64_t h, uint64_t v) {
    h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
    h *= 0xff51afd7ed558ccdull;
    h ^= h >> 33;
    return h;
}

__global__ __launch_bounds__(kAdvBlock) void prompt_hash_kernel(const int64_t* prompts, int64_t len, int64_t stride,
                                                                uint64_t* hashes) {
    __shared__ uint64_t sm[kAdvWaves];
    const int64_t b = blockIdx.x;
    const int64_t* row = prompts + b * stride;
    // position-dependent per-element hash, combined with a commutative sum
    uint64_t h = 0;
    for (int64_t i = threadIdx.x; i < len; i += kAdvBlock) h += mix64(static_cast<uint64_t>(i) * 0x100000001b3ull + 1, static_cast<uint64_t>(row[i]));
    h = block_sum<uint64_t, kAdvWaves>(h, sm);
    if (threadIdx.x == 0) hashes[b] = h;
}

__global__ __launch_bounds__(kAdvBlock) void prompt_group_kernel(const int64_t* prompts, int64_t len, int64_t stride,
                                                                 const uint64_t* hashes, int32_t* group) {
    __shared__ int sm_flag[kAdvWaves];
    const int64_t b = blockIdx.x;
    const uint64_t hb = hashes[b];
    const int64_t* row = prompts + b * stride;
    int32_t rep = static_cast<int32_t>(b);
    for (int64_t j = 0; j < b; ++j) {
        if (hashes[j] != hb) continue;  // uniform across the workgroup
        const int64_t* other = prompts + j * stride;
        int differs = 0;
        for (int64_t i = threadIdx.x; i < len; i += kAdvBlock) differs |= (row[i] != other[i]);
        if (block_sum<int, kAdvWaves>(differs, sm_flag) == 0) { rep = static_cast<int32_t>(j); break; }
    }
    if (threadIdx.x == 0) group[b] = rep;
}

__global__ void group_stats_kernel(const int32_t* group, int64_t batch, const float* rewards, const float* valid,
                                   const float* std_rewards, int loo, int normalize, float* baseline, float* stdv,
                                   float* adv) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= batch) return;
    const int32_t g = group[i];
    const float* sr = std_rewards ? std_rewards : rewards;
    float n_valid = 0.f, s1 = 0.f, s1s = 0.f, s2 = 0.f;
    for (int64_t j = 0; j < batch; ++j) {
        if (group[j] != g) continue;
        const float v = valid[j];
        n_valid += v;
        if (loo && j == i) continue;  // (1 - I) row of the mixing matrix
        s1 += rewards[j] * v;
        s1s += sr[j] * v;
        s2 += (sr[j] * sr[j]) * v;
    }
    float base, sd = 0.f;
    if (n_valid <= 1.f) {
        base = rewards[i];
    } else {
        const float n = n_valid - static_cast<float>(loo);
        base = s1 / n;
        const float e1 = s1s / n, e2 = s2 / n;
        sd = sqrtf((e2 - e1 * e1) * (n / (n - 1.f)));
        if (sd != sd) sd = 0.f;                      // nan_to_num(0): NaN -> 0,
        else if (sd == INFINITY) sd = FLT_MAX;       // +inf -> largest finite value
    }
    baseline[i] = base;
    stdv[i] = sd;
    if (adv) {
        float a = rewards[i] - base;
        if (normalize && sd > 0.f) a = a / (sd + 1e-6f);
        adv[i] = a;
    }
}

// ---------------------------------------------------------------------------------------------
// Per-sequence multiplicative logprob error between the generation engine and the policy, and the mask
// that drops sequences above a threshold.  Launch 1: one workgroup per sequence.  Launch 2: one workgroup
// reduces the sequences in a fixed order into an 8-float record.
// ---------------------------------------------------------------------------------------------
struct SeqErrArgs {
    const float* prev;   // [B, S] row stride prev_stride; column 0 is skipped
    const float* gen;
    const float* token_mask;
    const float* sample_mask;  // [B]
    const float* rewards;      // [B] or NULL
    int64_t batch, seq_len, prev_stride, gen_stride, tm_stride;
    int has_threshold;
    float threshold;
    float* seq_err;          // [B]
    float* valid;            // [B] 1 if the sequence has any unmasked token
    float* sample_mask_out;  // [B] (= sample_mask when no threshold)
    float* record;           // [8]
};

__global__ __launch_bounds__(kAdvBlock) void seq_err_rows_kernel(SeqErrArgs a) {
    __shared__ float sm[kAdvWaves];
    const int64_t b = blockIdx.x;
    const float smv = a.sample_mask[b];
    float num = 0.f, den = 0.f;
    for (int64_t t = 1 + threadIdx.x; t < a.seq_len; t += kAdvBlock) {
        const float m = a.token_mask[b * a.tm_stride + t] * smv;
        const float e = fabsf(a.gen[b * a.gen_stride + t] - a.prev[b * a.prev_stride + t]);
        num += expf(e * m) * m;
        den += m;
    }
    num = block_sum<float, kAdvWaves>(num, sm);
    den = block_sum<float, kAdvWaves>(den, sm);
    if (threadIdx.x == 0) {
        const bool valid = den > 0.f;
        const float err = valid ? num / fmaxf(den, 1.f) : 0.f;
        a.seq_err[b] = err;
        a.valid[b] = valid ? 1.f : 0.f;
        a.sample_mask_out[b] = a.has_threshold ? ((err <= a.threshold) ? 1.f : 0.f) * smv : smv;
    }
}

__global__ __launch_bounds__(kAdvBlock) void seq_err_finish_kernel(SeqErrArgs a) {
    __shared__ float sm[kAdvWaves];
    float mx = -FLT_MAX, mn = FLT_MAX, sum = 0.f, cnt = 0.f;
    float mx2 = -FLT_MAX, mn2 = FLT_MAX, sum2 = 0.f, cnt2 = 0.f, n_masked = 0.f, n_correct = 0.f;
    for (int64_t b = threadIdx.x; b < a.batch; b += kAdvBlock) {
        const float e = a.seq_err[b];
        const bool valid = a.valid[b] != 0.f;
        if (valid) { mx = fmaxf(mx, e); mn = fminf(mn, e); sum += e; cnt += 1.f; }
        if (a.has_threshold) {
            const float kept = a.sample_mask_out[b], diff = a.sample_mask[b] - kept;
            n_masked += diff;
            if (diff != 0.f && a.rewards && a.rewards[b] == 1.f) n_correct += 1.f;
            if (kept != 0.f && valid) { mx2 = fmaxf(mx2, e); mn2 = fminf(mn2, e); sum2 += e; cnt2 += 1.f; }
        }
    }
    mx = block_max<kAdvWaves>(mx, sm); mn = block_min<kAdvWaves>(mn, sm);
    sum = block_sum<float, kAdvWaves>(sum, sm); cnt = block_sum<float, kAdvWaves>(cnt, sm);
    mx2 = block_max<kAdvWaves>(mx2, sm); mn2 = block_min<kAdvWaves>(mn2, sm);
    sum2 = block_sum<float, kAdvWaves>(sum2, sm); cnt2 = block_sum<float, kAdvWaves>(cnt2, sm);
    n_masked = block_sum<float, kAdvWaves>(n_masked, sm); n_correct = block_sum<float, kAdvWaves>(n_correct, sm);
    if (threadIdx.x == 0) {
        float* r = a.record;
        r[0] = cnt > 0.f ? mx : 0.f;
        r[1] = cnt > 0.f ? sum / cnt : 0.f;
        r[2] = cnt > 0.f ? mn : 0.f;
        if (a.has_threshold) {
            r[3] = cnt2 > 0.f ? mx2 : 0.f;
            r[4] = cnt2 > 0.f ? sum2 / cnt2 : 0.f;
            r[5] = cnt2 > 0.f ? mn2 : 0.f;
        } else {
            r[3] = r[0]; r[4] = r[1]; r[5] = r[2];
        }
        const int masked = static_cast<int>(n_masked);  // the reference truncates the float sum the same way
        r[6] = static_cast<float>(masked);
        r[7] = masked > 0 ? n_correct / static_cast<float>(masked) : 0.f;
    }
}

// ---------------------------------------------------------------------------------------------
// Indices of the non-zero entries of a vector, ascending: the prompt groups that dynamic sampling keeps
// (std != 0).  One workgroup walks the vector 256 entries at a time; a wave's ballot and the waves'
// running counts give every kept entry its output slot, so the order of the input is preserved.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kAdvBlock) void nonzero_indices_kernel(const float* v, int64_t n, int32_t* idx, int32_t* count) {
    __shared__ int wave_cnt[kAdvWaves];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int base = 0;
    for (int64_t i0 = 0; i0 < n; i0 += kAdvBlock) {
        const int64_t i = i0 + threadIdx.x;
        const bool keep = i < n && v[i] != 0.0f;  // NaN != 0 is true, as in the reference's `std != 0.0`
        const unsigned long long ballot = __ballot(keep);
        if (lane == 0) wave_cnt[wave] = __popcll(ballot);
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kAdvWaves; ++w) {
            before += w < wave ? wave_cnt[w] : 0;
            total += wave_cnt[w];
        }
        if (keep) idx[base + before + __popcll(ballot & ((1ull << lane) - 1ull))] = static_cast<int32_t>(i);
        base += total;
        __syncthreads();
    }
    if (threadIdx.x == 0) *count = base;
}

}  // namespace nrl

using namespace nrl;

extern "C" int nrl_nonzero_indices(const float* values, int64_t n, int32_t* indices_out, int32_t* count_out, void* stream) {
    if (n < 0 || n >= (1ll << 31)) return fail(NRL_E_INVALID, "bad length %lld", (long long)n);
    if (!count_out || (n > 0 && (!values || !indices_out))) return fail(NRL_E_INVALID, "null argument");
    nonzero_indices_kernel<<<dim3(1), dim3(kAdvBlock), 0, static_cast<hipStream_t>(stream)>>>(values, n, indices_out, count_out);
    return check_launch("nonzero_indices");
}

extern "C" int64_t nrl_group_workspace_bytes(int64_t batch) {
    const int64_t b = batch < 1 ? 1 : batch;
    return b * static_cast<int64_t>(sizeof(uint64_t)) + b * static_cast<int64_t>(sizeof(int32_t));
}

extern "C" int nrl_group_baseline_std(const int64_t* prompts, int64_t batch, int64_t prompt_len, int64_t prompt_stride,
                                      const float* rewards, const float* valid, const float* std_rewards,
                                      int32_t leave_one_out, int32_t normalize, float* baseline_out, float* std_out,
                                      float* adv_out, int32_t* group_out, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
    if (batch < 0 || prompt_len < 0) return fail(NRL_E_INVALID, "bad shape [%lld, %lld]", (long long)batch, (long long)prompt_len);
    if (batch == 0) return NRL_OK;
    if (batch >= (1ll << 31)) return fail(NRL_E_INVALID, "batch too large");
    if ((prompt_len > 0 && !prompts) || !rewards || !valid || !baseline_out || !std_out || !workspace)
        return fail(NRL_E_INVALID, "null argument");
    if (workspace_bytes < nrl_group_workspace_bytes(batch)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 7) return fail(NRL_E_INVALID, "workspace must be 8-byte aligned");
    uint64_t* hashes = static_cast<uint64_t*>(workspace);
    int32_t* group = group_out ? group_out : reinterpret_cast<int32_t*>(hashes + batch);
    hipStream_t s = static_cast<hipStream_t>(stream);
    prompt_hash_kernel<<<dim3((unsigned)batch), dim3(kAdvBlock), 0, s>>>(prompts, prompt_len, prompt_stride, hashes);
    prompt_group_kernel<<<dim3((unsigned)batch), dim3(kAdvBlock), 0, s>>>(prompts, prompt_len, prompt_stride, hashes, group);
    group_stats_kernel<<<dim3((unsigned)((batch + 127) / 128)), dim3(128), 0, s>>>(
        group, batch, rewards, valid, std_rewards, leave_one_out, normalize, baseline_out, std_out, adv_out);
    return check_launch("group_baseline_std");
}

extern "C" int nrl_seq_logprob_error(const float* prev, int64_t prev_stride, const float* gen, int64_t gen_stride,
                                     const float* token_mask, int64_t token_mask_stride, const float* sample_mask,
                                     const float* rewards, int64_t batch, int64_t seq_len, int32_t has_threshold,
                                     float threshold, float* seq_err_out, float* sample_mask_out, float* record_out,
                                     void* workspace, int64_t workspace_bytes, void* stream) {
    if (batch < 0 || seq_len < 0) return fail(NRL_E_INVALID, "bad shape");
    if (!record_out) return fail(NRL_E_INVALID, "record_out is NULL");
    if (batch > 0 && (!prev || !gen || !token_mask || !sample_mask || !seq_err_out || !sample_mask_out || !workspace))
        return fail(NRL_E_INVALID, "null argument");
    if (workspace_bytes < batch * static_cast<int64_t>(sizeof(float))) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (batch >= (1ll << 31)) return fail(NRL_E_INVALID, "too many sequences");
    SeqErrArgs a;
    a.prev = prev; a.gen = gen; a.token_mask = token_mask; a.sample_mask = sample_mask; a.rewards = rewards;
    a.batch = batch; a.seq_len = seq_len; a.prev_stride = prev_stride; a.gen_stride = gen_stride; a.tm_stride = token_mask_stride;
    a.has_threshold = has_threshold; a.threshold = threshold;
    a.seq_err = seq_err_out; a.valid = static_cast<float*>(workspace); a.sample_mask_out = sample_mask_out; a.record = record_out;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (batch > 0) seq_err_rows_kernel<<<dim3((unsigned)batch), dim3(kAdvBlock), 0, s>>>(a);
    seq_err_finish_kernel<<<dim3(1), dim3(kAdvBlock), 0, s>>>(a);
    return check_launch("seq_logprob_error");
}

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

__global__ __launch_bounds__(kAdvBlock) void prompt_group_kernel(const int64_t* prompts, int64_t batch, int64_t len,
                                                                 int64_t stride, const uint64_t* hashes, int32_t* group) {
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

}  // namespace nrl

using namespace nrl;

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
    prompt_group_kernel<<<dim3((unsigned)batch), dim3(kAdvBlock), 0, s>>>(prompts, batch, prompt_len, prompt_stride, hashes, group);
    group_stats_kernel<<<dim3((unsigned)((batch + 127) / 128)), dim3(128), 0, s>>>(
        group, batch, rewards, valid, std_rewards, leave_one_out, normalize, baseline_out, std_out, adv_out);
    return check_launch("group_baseline_std");
}

// K3: token logprobs under top-k / top-p (nucleus) filtering, forward and backward, for gfx950.
//
// The reference sorts every 151 936-wide row (values + int64 indices).  Here one workgroup of 256
// threads owns a row and never sorts it:
//   pass 1 (HBM)   streams the row keeping 2048 chunk maxima in registers (and, when the caller
//                  wants the unfiltered logprob too, the online log-sum-exp of the full row); a chunk
//                  is a set of whole 128-byte lines, so that what pass 2 re-reads is all used;
//   select         the k-th largest chunk maximum is a lower bound of the k-th largest element
//                  (found two bits per round with wave ballots, the maxima staying in registers);
//                  for top-p alone the bound starts at lse + log((1-p)/V) (everything below it is
//                  dropped whatever the order) and is raised with a 64-bin histogram of probability
//                  over log-probability, filled from the chunk maxima and, only if that is not
//                  enough, from the row read once more;
//   pass 2         re-reads only the chunks whose maximum reaches the bound (about k of 2048) and
//                  appends the elements above the bound to an LDS list;
//   finish         bitonic sort of the list by (value, index), top-k threshold with ties kept,
//                  softmax over the kept values, ascending cumulative mass > 1 - top_p, the
//                  renormalised log-sum-exp, the target's logprob (-inf when it was filtered).
// Per row the forward saves (threshold value, tie index, kept log-sum-exp): element v is kept iff
// x_v > thr, or x_v == thr and v >= tie index.  Among exactly tied values at the top-p boundary the
// larger vocabulary indices survive (ascending stable order); all ties at the top-k threshold are
// kept.  The backward streams the row once more: d_v = keep_v * g * (onehot_v - exp(x_v - lse_kept)).
//
// Rows whose candidate list would exceed the LDS capacity (very flat distributions under top-p
// alone, thousands of exact ties, or a top_k in the thousands) are marked and finished by
// topk_topp_wide_kernel, which finds the same predicate by a radix descent over the row's order keys
// (a histogram pass per key digit: two to three passes for 16-bit logits).

#include <float.h>
#include <math.h>

#include <type_traits>

#include "common.hpp"

namespace nrl {

constexpr int kSelBlock = 256;
constexpr int kSelWaves = kSelBlock / kWave;
constexpr int kMassBins = 64;
constexpr int kLooseHits = 768;  // top-p alone: more hit chunks than this under the chunk maxima's bound -> bound from the row
constexpr int kMassCopies = 8;  // copies of the histogram, by lane: most elements fall into the few lowest bins
constexpr int kWideGrid = 2048;  // workgroups of the kernel that finishes the marked rows
constexpr int32_t kTieUnresolved = -1;  // tie[] marker: the row's kept set did not fit the candidate list
constexpr int kSub = 8;                      // chunk maxima per thread
constexpr int kChunks = kSelBlock * kSub;    // 2048
constexpr int kCap = 4096;                   // candidate capacity (LDS); rows under a small top-k use kCapSmall
constexpr int kCapSmall = 2048;              // ... which lets six workgroups share a compute unit instead of three
constexpr int kSmallTopK = 512;

struct Lse2 {
    float m, s;
};
__device__ __forceinline__ Lse2 lse2_merge(Lse2 a, Lse2 b) {
    const float m = fmaxf(a.m, b.m);
    Lse2 r;
    r.m = m;
    r.s = a.s * fast_exp2((a.m - m) * kLog2e) + b.s * fast_exp2((b.m - m) * kLog2e);
    return r;
}

// monotone map float -> uint32 (larger float, larger key)
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// maximum over the 8 consecutive lanes (aligned to 8) that read one 128-byte line; every lane returns it
// (written as three hand-placed v_max_f32_dpp the pass has a third fewer vector instructions and takes the same time)
__device__ __forceinline__ float line_max(float v) {
    int x = __float_as_int(v);
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false)));   // quad_perm [1,0,3,2]
    x = __float_as_int(v);
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false)));   // quad_perm [2,3,0,1]
    x = __float_as_int(v);
    return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x141, 0xF, 0xF, false)));  // row_half_mirror
}

template <int DT> __device__ __forceinline__ int64_t sel_row_head(const void* row, int64_t vocab) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(row);
    const int64_t h = static_cast<int64_t>(((16 - (a & 15)) & 15) / Row<DT>::BYTES);
    return h < vocab ? h : vocab;
}

template <int CAP> struct SelShared {
    unsigned long long cand[CAP];
    float expv[CAP];
    int sel_cnt[2][kSelWaves * 3];
    Lse2 lse_w[kSelWaves];
    int count;
    float mass_bin[kMassCopies * kMassBins];  // top-p alone: probability mass per log-probability bin
    int n_hit;  // chunks whose maximum reaches the bound (their list lives in expv until the finish phase)
};

// k-th largest (1-based) of the workgroup's kChunks keys (kSub per thread, in registers); every thread
// returns it.  Two bits at a time from the top: the answer is the largest v with at least k keys >= v.  A
// round costs 3 * kSub ballots per wave, three LDS words per wave and one barrier (the buffers alternate), with
// no atomics -- chunk maxima share their high bits, so a histogram would serialise on one bin.
template <int CAP>
__device__ __forceinline__ uint32_t select_kth_largest(SelShared<CAP>& sh, const uint32_t (&keys)[kSub], int k) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    uint32_t v = 0u;
    for (int bit = 30; bit >= 0; bit -= 2) {  // two bits per round: three trial values, one barrier
        int cnt[3] = {0, 0, 0};
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            const uint32_t cand = v | (static_cast<uint32_t>(c + 1) << bit);
#pragma unroll
            for (int u = 0; u < kSub; ++u) cnt[c] += __popcll(__ballot(keys[u] >= cand));
        }
        const int par = (bit >> 1) & 1;
        if (lane < 3) sh.sel_cnt[par][wave * 3 + lane] = lane == 0 ? cnt[0] : lane == 1 ? cnt[1] : cnt[2];
        __syncthreads();
        int tot[3] = {0, 0, 0};
#pragma unroll
        for (int w = 0; w < kSelWaves; ++w)
#pragma unroll
            for (int c = 0; c < 3; ++c) tot[c] += sh.sel_cnt[par][w * 3 + c];
        // counts fall as the trial value rises: take the largest trial that still has k keys at or above it
        const uint32_t step = tot[2] >= k ? 3u : tot[1] >= k ? 2u : tot[0] >= k ? 1u : 0u;
        v |= step << bit;
    }
    return v;
}

// sum of e[n-1], e[n-2], ..., e[0] in exactly that order; called by every lane of one wave, which all
// return the same value (64 elements per LDS read, then lane-to-scalar moves instead of one dependent
// LDS round trip per element)
__device__ __forceinline__ float wave_seq_sum_desc(const float* e, int n) {
    const int lane = threadIdx.x & (kWave - 1);
    float s = 0.f;
    for (int blk = (n - 1) / kWave; blk >= 0; --blk) {
        const int idx = blk * kWave + lane;
        // lanes past the end hold 0 and come first in this order, where adding them changes nothing; with a
        // fixed trip count the loop unrolls into 64 lane reads with constant indices
        const float v = idx < n ? e[idx] : 0.f;
#pragma unroll
        for (int i = kWave - 1; i >= 0; --i) s += __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), i));
    }
    return s;
}

// descending bitonic sort of sh.cand[0 .. n_pad)
template <int CAP> __device__ __forceinline__ void sort_candidates_desc(SelShared<CAP>& sh, int n_pad) {
    const int tid = threadIdx.x;
    if (n_pad <= 2 * kWave) {
        // short lists (the usual case under top-k) are sorted by one wave alone: its LDS operations execute
        // in order, so the compare-exchange steps need no workgroup barrier
        __syncthreads();
        if (tid < kWave) {
            for (int size = 2; size <= n_pad; size <<= 1) {
                for (int stride = size >> 1; stride > 0; stride >>= 1) {
                    const int i = tid;
                    if (i < (n_pad >> 1)) {
                        const int lo = ((i / stride) * (stride << 1)) + (i % stride);
                        const int hi = lo + stride;
                        const bool desc = ((lo & size) == 0);
                        const unsigned long long a = sh.cand[lo], b = sh.cand[hi];
                        if ((a < b) == desc) { sh.cand[lo] = b; sh.cand[hi] = a; }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                }
            }
        }
        __syncthreads();
        return;
    }
    for (int size = 2; size <= n_pad; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int i = tid; i < (n_pad >> 1); i += kSelBlock) {
                const int lo = ((i / stride) * (stride << 1)) + (i % stride);
                const int hi = lo + stride;
                const bool desc = ((lo & size) == 0);
                const unsigned long long a = sh.cand[lo], b = sh.cand[hi];
                if ((a < b) == desc) { sh.cand[lo] = b; sh.cand[hi] = a; }
            }
        }
    }
    __syncthreads();
}

struct SelArgs {
    const void* logits;
    int64_t n_inner, vocab, stride_outer, stride_inner;
    const int64_t* targets;  // may be NULL (filter only)
    int64_t ts_outer, ts_inner;
    float tparam;
    int top_k;    // <= 0: off
    float top_p;  // >= 1: off
    float* logprob;      // [rows] or NULL
    float* thr;          // [rows]
    int32_t* tie;        // [rows]
    float* lse_kept;     // [rows]
    float* logprob_full; // [rows] or NULL: unfiltered logprob of the target
    float* lse_full;     // [rows] or NULL
    // the kept set itself, for a backward that does not read the row again (all three NULL: not recorded):
    int32_t* kept_n;     // [rows] number of kept elements, -1 if they do not fit kept_cap (or the row was left to the wide kernel)
    int32_t* kept_idx;   // [rows, kept_cap] their vocabulary indices, in descending (value, index) order
    float* kept_x;       // [rows, kept_cap] their (scaled) logits
    int kept_cap;
};

// PONLY: top-p without top-k (its own instantiation, so that the mass histogram costs the top-k variants
// neither registers nor LDS); otherwise top-k is on, with or without top-p.
template <int DT, int TEMP, bool FULL_LSE, int CAP, bool PONLY = false>
__global__ __launch_bounds__(kSelBlock) void topk_topp_fwd_kernel(SelArgs a) {
    static_assert(!PONLY || FULL_LSE, "top-p alone normalises over the whole row");
    __shared__ SelShared<CAP> sh;
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const int64_t r = blockIdx.x;
    const int64_t o = r / a.n_inner, i_in = r - o * a.n_inner;
    const char* row = static_cast<const char*>(a.logits) + (o * a.stride_outer + i_in * a.stride_inner) * Row<DT>::BYTES;
    const int64_t vocab = a.vocab;
    const int64_t head = sel_row_head<DT>(row, vocab);
    const int64_t nvec = (vocab - head) / EPV;
    const int64_t tail0 = head + nvec * EPV;
    const u32x4* xv = reinterpret_cast<const u32x4*>(row + head * Row<DT>::BYTES);

    // ---- pass 1: chunk maxima (+ full-row online log-sum-exp) ----
    // Without the full-row log-sum-exp only maxima leave this pass, and the temperature scaling (a multiplication or
    // division by a positive number, then rounding to the logits' dtype) is monotone: the maximum of the scaled
    // values is the scaled maximum, so the raw values are compared and each chunk maximum is scaled once at the end.
    constexpr bool LATE_SCALE = !FULL_LSE && TEMP != 0;
    auto scaled = [&](float x) { return LATE_SCALE ? x : scale_logit<DT, TEMP>(x, a.tparam); };
    float mx[kSub];
#pragma unroll
    for (int u = 0; u < kSub; ++u) mx[u] = -FLT_MAX;
    Lse2 acc;
    acc.m = -FLT_MAX;
    acc.s = 0.f;
    // A chunk is a set of whole 128-byte lines: the 8 lanes that read one line together reduce their maxima over
    // the line, and lane j of the 8 keeps the lines of the iterations i with i % 8 == j.  The second pass then
    // re-reads full lines; with a chunk per thread it re-read 16 bytes of a line at a time, and every such piece
    // cost the whole line in HBM traffic.
    const int lane8 = tid & 7;
    int64_t base = 0;
    int iter = 0;
    for (; base + kSub * kSelBlock <= nvec; base += kSub * kSelBlock, ++iter) {
        u32x4 q[kSub];
#pragma unroll
        for (int u = 0; u < kSub; ++u) q[u] = __builtin_nontemporal_load(xv + base + u * kSelBlock + tid);
        const bool mine = (iter & 7) == lane8;
        float v[kSub * EPV];
        float vm_all = -FLT_MAX;
#pragma unroll
        for (int u = 0; u < kSub; ++u) {
            float t[EPV];
            Row<DT>::decode(q[u], t);
            float vm = -FLT_MAX;
#pragma unroll
            for (int k = 0; k < EPV; ++k) {
                t[k] = scaled(t[k]);
                v[u * EPV + k] = t[k];
                vm = fmaxf(vm, t[k]);
            }
            vm_all = fmaxf(vm_all, vm);
            const float lm = line_max(vm);
            mx[u] = fmaxf(mx[u], mine ? lm : -FLT_MAX);
        }
        if (FULL_LSE) {
            const float mn = fmaxf(acc.m, vm_all);
            float part = 0.f;
#pragma unroll
            for (int k = 0; k < kSub * EPV; ++k) part += fast_exp2((v[k] - mn) * kLog2e);
            acc.s = acc.s * fast_exp2((acc.m - mn) * kLog2e) + part;
            acc.m = mn;
        }
    }
    // the ragged end of the row, one more iteration with fewer than kSub vectors per thread: the same chunks
    {
        const bool mine = (iter & 7) == lane8;
#pragma unroll
        for (int u = 0; u < kSub; ++u) {
            const int64_t vi = base + u * kSelBlock + tid;
            float vm = -FLT_MAX;
            if (vi < nvec) {
                float t[EPV];
                Row<DT>::decode(xv[vi], t);
#pragma unroll
                for (int k = 0; k < EPV; ++k) {
                    t[k] = scaled(t[k]);
                    vm = fmaxf(vm, t[k]);
                    if (FULL_LSE) {
                        const float mn = fmaxf(acc.m, t[k]);
                        acc.s = acc.s * fast_exp2((acc.m - mn) * kLog2e) + fast_exp2((t[k] - mn) * kLog2e);
                        acc.m = mn;
                    }
                }
            }
            const float lm = line_max(vm);  // by every lane: lanes past the end bring the identity
            mx[u] = fmaxf(mx[u], mine ? lm : -FLT_MAX);
        }
    }
    {
        const int64_t e0 = tid < head ? tid : -1;
        const int64_t e1 = tail0 + tid < vocab ? tail0 + tid : -1;
        for (int w = 0; w < 2; ++w) {
            const int64_t e = w == 0 ? e0 : e1;
            if (e < 0) continue;
            const float x = scaled(Row<DT>::load1(row, e));
            mx[0] = fmaxf(mx[0], x);
            if (FULL_LSE) {
                const float mn = fmaxf(acc.m, x);
                acc.s = acc.s * fast_exp2((acc.m - mn) * kLog2e) + fast_exp2((x - mn) * kLog2e);
                acc.m = mn;
            }
        }
    }
    if (LATE_SCALE) {
#pragma unroll
        for (int u = 0; u < kSub; ++u) mx[u] = scale_logit<DT, TEMP>(mx[u], a.tparam);
    }
    uint32_t mx_key[kSub];
#pragma unroll
    for (int u = 0; u < kSub; ++u) mx_key[u] = order_key(mx[u]);
    float lse_full = 0.f;
    if (FULL_LSE) {
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            Lse2 other;
            other.m = __shfl_xor(acc.m, off, kWave);
            other.s = __shfl_xor(acc.s, off, kWave);
            acc = lse2_merge(acc, other);
        }
        if ((tid & (kWave - 1)) == 0) sh.lse_w[tid / kWave] = acc;
    }
    if (tid == 0) { sh.count = 0; sh.n_hit = 0; }
    __syncthreads();
    if (FULL_LSE) {
        Lse2 tot = sh.lse_w[0];
#pragma unroll
        for (int w = 1; w < kSelWaves; ++w) tot = lse2_merge(tot, sh.lse_w[w]);
        lse_full = tot.m + logf(tot.s);
    }

    // ---- lower bound of everything that can be kept ----
    constexpr bool use_k = !PONLY;
    const bool use_p = a.top_p < 1.0f;
    uint32_t bound_key = 0u;
    // top-p alone: elements with probability <= (1-p)/V sum to at most 1-p and are the smallest, which puts
    // a first bound b0 under the kept set; but a long tail leaves thousands of elements above b0.  The
    // probability of a set of elements above b0, sorted into kMassBins equal log-probability bins, gives a
    // better one: if the bins from j upwards already hold more than p of the row's mass, everything below
    // bin j weighs less than 1-p and cannot be kept.  First the set is the 2048 chunk maxima (already in
    // registers; enough whenever the kept set is a few hundred tokens), and only if that proves nothing or
    // leaves too many candidates the whole row, read once more.
    const float cut = 1.0f - a.top_p;
    const float span = logf(static_cast<float>(vocab) / cut);  // from probability (1-p)/V up to 1, in nats
    const float b0 = lse_full - span;
    // The bins start a quarter of the span above b0: an edge lower than that would keep thousands of tokens,
    // more than the list holds anyway, and the many elements just above b0 would each cost an LDS atomic.
    const float hb = b0 + 0.25f * span;
    const float to_bin = static_cast<float>(kMassBins) / (0.75f * span);
    auto bin = [&](float x) {
        if (x > hb) {
            const int j = static_cast<int>((x - hb) * to_bin);
            atomicAdd(&sh.mass_bin[(tid & (kMassCopies - 1)) * kMassBins + (j < kMassBins - 1 ? j : kMassBins - 1)], expf(x - lse_full));
        }
    };
    // called by every thread between two barriers around the binning; returns the bound (the same in all)
    auto bound_from_bins = [&]() -> uint32_t {
        // every wave: lane j takes bin j and the mass of the bins from j upwards.  The highest edge whose
        // mass below stays under 1-p (less a margin for the rounding of the sums: the list may hold more
        // than the kept set, never less) bounds the candidates; with none the bound stays at b0.
        static_assert(kMassBins == kWave, "one bin per lane");
        float above = 0.f;
#pragma unroll
        for (int q = 0; q < kMassCopies; ++q) above += sh.mass_bin[q * kMassBins + (tid & (kWave - 1))];
#pragma unroll
        for (int off = 1; off < kWave; off <<= 1) {
            const float up = __shfl_down(above, off, kWave);
            if ((tid & (kWave - 1)) + off < kWave) above += up;
        }
        const unsigned long long ok = __ballot(1.0f - above <= cut * 0.999f - 1e-5f);
        const int edge = ok ? 63 - __builtin_clzll(ok) : 0;
        // just under the edge, so that an element the rounding of its bin number put into bin `edge` counts
        return ok ? order_key(hb + (static_cast<float>(edge) - 0.01f) / to_bin) : order_key(b0) + 1u;
    };
    auto clear_bins = [&]() {
        for (int i = tid; i < kMassCopies * kMassBins; i += kSelBlock) sh.mass_bin[i] = 0.f;
    };
    auto bound_from_row = [&]() -> uint32_t {
        clear_bins();
        __syncthreads();
        for (int64_t vb = 0; vb < nvec; vb += kSub * kSelBlock) {  // kSub loads in flight per thread
            u32x4 q[kSub];
#pragma unroll
            for (int u = 0; u < kSub; ++u) {
                const int64_t vi = vb + u * kSelBlock + tid;
                if (vi < nvec) q[u] = xv[vi];
            }
#pragma unroll
            for (int u = 0; u < kSub; ++u) {
                if (vb + u * kSelBlock + tid >= nvec) continue;
                float t[EPV];
                Row<DT>::decode(q[u], t);
#pragma unroll
                for (int k = 0; k < EPV; ++k) bin(scale_logit<DT, TEMP>(t[k], a.tparam));
            }
        }
        if (tid < head) bin(scale_logit<DT, TEMP>(Row<DT>::load1(row, tid), a.tparam));
        if (tail0 + tid < vocab) bin(scale_logit<DT, TEMP>(Row<DT>::load1(row, tail0 + tid), a.tparam));
        __syncthreads();
        return bound_from_bins();
    };
    bool whole_row = true;  // top-p alone: the bound already rests on the whole row
    bool force_wide = false;  // top-p alone: the chunk maxima show that the kept set cannot fit the candidate list
    if (use_k) {
        if (a.top_k <= kChunks) bound_key = select_kth_largest(sh, mx_key, a.top_k);
    } else {
        clear_bins();
        // (how many elements the chunks hold whose maxima fall into each bin, and what they would weigh if each
        // weighed as much as its chunk's maximum, is summed too, in integers: see below)
        int* max_cnt = reinterpret_cast<int*>(sh.cand);  // the candidate list is not in use yet
        unsigned long long* max_w = sh.cand + kMassBins;  // 32.32 fixed point
        if (tid <= kMassBins) { max_cnt[tid] = 0; max_w[tid] = 0ull; }
        __syncthreads();
        {
            // this lane's chunks are the lines of the iterations i = lane8, lane8 + 8, ... <= n_full (the ragged last
            // iteration counted whole); chunk 0 also took one element of the unaligned head and of the tail
            const int n_full_iter = static_cast<int>(nvec / (kSub * kSelBlock));
            const int lines = n_full_iter >= lane8 ? (n_full_iter - lane8) / 8 + 1 : 0;
#pragma unroll
            for (int u = 0; u < kSub; ++u) {
                bin(mx[u]);
                const int elems = lines * 8 * EPV + (u == 0 ? 2 : 0);
                int j = kMassBins;  // maxima under the first bin's lower edge
                if (mx[u] > hb) {
                    j = static_cast<int>((mx[u] - hb) * to_bin);
                    j = j < kMassBins - 1 ? j : kMassBins - 1;
                }
                atomicAdd(&max_cnt[j], elems);
                const float w = expf(fminf(mx[u] - lse_full, 0.f)) * 4294967296.0f;  // NaN (no finite row sum) -> 0
                atomicAdd(&max_w[j], static_cast<unsigned long long>(w) * static_cast<unsigned long long>(elems));
            }
        }
        __syncthreads();
        bound_key = bound_from_bins();
        whole_row = bound_key == order_key(b0) + 1u;  // the maxima alone prove nothing: go to the row at once
        if (whole_row) {
            // A row whose kept set cannot fit the candidate list is not worth the two passes that would find that
            // out.  No element outweighs the maximum of its chunk, so the CAP heaviest elements of the row weigh at
            // most what all elements of the chunks with the heaviest maxima would, taken chunk by chunk until CAP
            // elements are reached, each at its chunk's maximum; if even that stays under top_p, more than CAP
            // elements are kept and the row goes to the wide kernel now.  Counts and weights are summed as integers,
            // so the decision does not depend on the order in which atomics arrived (both paths find the same kept
            // set up to near-equal elements at the boundary, but a row should take the same path every time).
            static_assert(kMassBins == kWave, "one bin per lane");
            const int lane_b = tid & (kWave - 1);
            int c_above = max_cnt[lane_b];   // becomes: elements of the chunks whose maxima lie in bins >= lane_b
            unsigned long long w_above = max_w[lane_b];  // their weight, each element at its chunk's maximum
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                const int cu = __shfl_down(c_above, off, kWave);
                const unsigned long long wu = __shfl_down(w_above, off, kWave);
                if (lane_b + off < kWave) { c_above += cu; w_above += wu; }
            }
            const unsigned long long enough = __ballot(c_above >= CAP);
            const int jstar = enough ? 63 - __builtin_clzll(enough) : 0;
            const float w_star = static_cast<float>(__shfl(w_above, jstar, kWave)) * (1.0f / 4294967296.0f);
            const int c_star = __shfl(c_above, jstar, kWave);
            // chunks whose maxima were not binned lie under hb
            float heaviest = w_star + static_cast<float>(c_star < CAP ? CAP - c_star : 0) * expf(hb - lse_full);
            if (enough) {
                // of bin jstar only as many elements as the list still has room for, each at the bin's upper edge
                const int up = jstar + 1 < kWave ? jstar + 1 : jstar;
                const unsigned long long w_up = __shfl(w_above, up, kWave);
                const int c_up = __shfl(c_above, up, kWave);
                const float w_next = jstar + 1 < kWave ? static_cast<float>(w_up) * (1.0f / 4294967296.0f) : 0.f;
                const int c_next = jstar + 1 < kWave ? c_up : 0;
                const float edge = jstar == kMassBins - 1 ? 0.f : fminf(hb + static_cast<float>(jstar + 1) / to_bin - lse_full, 0.f);
                heaviest = fminf(heaviest, w_next + static_cast<float>(CAP - c_next) * expf(edge));
            }
            force_wide = heaviest < 0.98f * a.top_p;
            if (!force_wide) {
                __syncthreads();  // every wave is done with the bins
                bound_key = bound_from_row();
            }
        }
    }

    // ---- pass 2: collect candidates (top-p alone: once more with the bound from the whole row if the list
    // did not hold what the chunk maxima's bound lets through) ----
    int n = force_wide ? CAP + 1 : 0;
    for (; !force_wide;) {
    // Only the chunks whose maximum reaches the bound can hold candidates (with top-k that is about k of the
    // 2048 chunks, a few percent of the row).
    auto push = [&](uint32_t key, int64_t index) {
        if (key >= bound_key) {
            const int pos = atomicAdd(&sh.count, 1);
            if (pos < CAP) sh.cand[pos] = (static_cast<unsigned long long>(key) << 32) | static_cast<uint32_t>(index);
        }
    };
    auto push_raw = [&](const u32x4& q, int64_t vi) {
        float t[EPV];
        Row<DT>::decode(q, t);
#pragma unroll
        for (int k = 0; k < EPV; ++k) push(order_key(scale_logit<DT, TEMP>(t[k], a.tparam)), head + vi * EPV + k);
    };
    // The hit chunks go to a list and their vectors are then dealt out evenly, a few per thread with the
    // loads in flight together: a thread that re-read only its own hit chunks left most lanes of a wave
    // idle through several thousand instructions, which cost more than the streaming pass.
    static_assert(kChunks <= 65536 && kChunks * 2 <= CAP * 4, "the hit list is 16-bit chunk ids inside expv");
    uint16_t* hit = reinterpret_cast<uint16_t*>(sh.expv);
#pragma unroll
    for (int u = 0; u < kSub; ++u)
        if (mx_key[u] >= bound_key) hit[atomicAdd(&sh.n_hit, 1)] = static_cast<uint16_t>(tid * kSub + u);
    if (mx_key[0] >= bound_key) {  // chunk 0 also took the unaligned head / tail elements
        if (tid < head) push(order_key(scale_logit<DT, TEMP>(Row<DT>::load1(row, tid), a.tparam)), tid);
        if (tail0 + tid < vocab)
            push(order_key(scale_logit<DT, TEMP>(Row<DT>::load1(row, tail0 + tid), a.tparam)), tail0 + tid);
    }
    __syncthreads();
    if (!use_k && !whole_row && sh.n_hit > kLooseHits) {
        // the bound from the chunk maxima lets too many chunks through: the row's own is worth its pass
        __syncthreads();  // every thread has read the hit count
        if (tid == 0) { sh.count = 0; sh.n_hit = 0; }
        whole_row = true;
        bound_key = bound_from_row();
        continue;
    }
    const int n_full = static_cast<int>(nvec / (kSub * kSelBlock));  // whole iterations of pass 1; number n_full is the ragged end
    const int per_chunk = ((n_full + 8) / 8) * 8;  // a line (8 vectors) per iteration the chunk's lane took
    const int n_items = sh.n_hit * per_chunk;
    // vector index of item number `item`, or -1 (an iteration past the end, or a vector past the row's)
    auto item_vec = [&](int item) -> int64_t {
        if (item >= n_items) return -1;
        const int h = item / per_chunk, rem = item - h * per_chunk;
        const int cu = hit[h], t = cu / kSub, u = cu - t * kSub;
        const int i = (t & 7) + (rem & ~7);  // iteration (rem / 8) of those with i % 8 == t % 8
        if (i > n_full) return -1;
        const int64_t vi = i * static_cast<int64_t>(kSub * kSelBlock) + u * kSelBlock + (t & ~7) + (rem & 7);
        return vi < nvec ? vi : -1;
    };
    constexpr int kBatch = 4;
    for (int i0 = tid; i0 < n_items; i0 += kBatch * kSelBlock) {
        // a list that has overflowed is not used (the bound is raised, or the row goes to the wide kernel): stop feeding
        // it -- on a flat row every element would otherwise queue up on the one counter
        if (*reinterpret_cast<volatile int*>(&sh.count) > CAP) break;
        int64_t vi[kBatch];
        u32x4 q[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            vi[j] = item_vec(i0 + j * kSelBlock);
            if (vi[j] >= 0) q[j] = xv[vi[j]];
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (vi[j] >= 0) push_raw(q[j], vi[j]);
    }
    __syncthreads();
    n = sh.count;
    if (use_k || whole_row || n <= CAP) break;
    __syncthreads();  // every thread has read the count
    if (tid == 0) { sh.count = 0; sh.n_hit = 0; }
    whole_row = true;
    bound_key = bound_from_row();
    }
    if (n > CAP || n == 0) {
        // the kept set does not fit the candidate list (or the row holds no finite value); the kernel that finishes
        // such a row finds its largest (scaled) logit in thr
        float row_max = mx[0];
#pragma unroll
        for (int u = 1; u < kSub; ++u) row_max = fmaxf(row_max, mx[u]);
        row_max = wave_max(row_max);
        __syncthreads();
        if ((tid & (kWave - 1)) == 0) sh.lse_w[tid / kWave].m = row_max;
        __syncthreads();
#pragma unroll
        for (int q = 0; q < kSelWaves; ++q) row_max = fmaxf(row_max, sh.lse_w[q].m);
        if (tid == 0) {
            a.thr[r] = n > CAP ? row_max : __builtin_nanf("");
            a.tie[r] = n > CAP ? kTieUnresolved : 0;  // unresolved rows are finished by topk_topp_wide_kernel
            a.lse_kept[r] = __builtin_nanf("");
            if (a.logprob) a.logprob[r] = __builtin_nanf("");
            if (a.lse_full) a.lse_full[r] = lse_full;
            if (a.logprob_full) a.logprob_full[r] = __builtin_nanf("");
            if (a.kept_n) a.kept_n[r] = -1;
        }
        return;
    }
    int n_pad = 1;
    while (n_pad < n) n_pad <<= 1;
    for (int i = n + tid; i < n_pad; i += kSelBlock) sh.cand[i] = 0ull;  // sorts last
    sort_candidates_desc(sh, n_pad);

    // ---- top-k threshold (ties kept), softmax over the kept values ----
    int n_k = n;
    if (use_k) {
        const int kk = a.top_k < n ? a.top_k : n;
        const uint32_t thr_key = static_cast<uint32_t>(sh.cand[kk - 1] >> 32);
        int cnt = 0;
        for (int i = tid; i < n; i += kSelBlock) cnt += (static_cast<uint32_t>(sh.cand[i] >> 32) >= thr_key) ? 1 : 0;
        __shared__ int cnt_w[kSelWaves];
        n_k = block_sum<int, kSelWaves>(cnt, cnt_w);
    }
    const float m = key_value(static_cast<uint32_t>(sh.cand[0] >> 32));
    for (int i = tid; i < n_k; i += kSelBlock)
        sh.expv[i] = expf(key_value(static_cast<uint32_t>(sh.cand[i] >> 32)) - m);
    __syncthreads();
    if (tid < kWave) {  // one wave; every lane computes the same scalars, lane 0 writes them
        int n_keep = n_k;
        if (use_p) {
            float s_k = wave_seq_sum_desc(sh.expv, n_k);
            // ascending cumulative probability, smallest kept value first; keep while it exceeds 1 - p
            const float cut = 1.0f - a.top_p;
            float cum = 0.f;
            if (!use_k) {
                // top-p alone normalises over the whole row: the elements below the candidate bound
                // come first in ascending order and contribute their (small) mass to the running sum
                const float s_full = expf(lse_full - m);
                cum = fmaxf(0.f, (s_full - s_k) / s_full);
                s_k = s_full;
            }
            // Elements fall, smallest first, while the running sum stays <= 1 - p; the sum only grows, so
            // counting the steps that end at or under the cut counts the fallen.  Whole blocks of 64 with
            // constant lane indices: lanes past the end come first and add nothing (each counts as a step
            // under the cut and is taken off again), index 0 is always kept and never enters the sum.
            const int top_blk = (n_k - 1) / kWave;
            int steps_under = 0;
            for (int blk = top_blk; blk >= 0; --blk) {
                const int idx = blk * kWave + tid;
                const float v = (idx >= 1 && idx < n_k) ? sh.expv[idx] / s_k : 0.f;
#pragma unroll
                for (int i = kWave - 1; i >= 0; --i) {
                    cum += __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), i));
                    steps_under += cum <= cut ? 1 : 0;
                }
                if (!(cum <= cut)) break;  // nothing further down can fall (also leaves on a NaN)
            }
            const int fallen = steps_under - ((top_blk + 1) * kWave - n_k);
            n_keep = n_k - fallen;
            if (n_keep < 1) n_keep = 1;
            if (n_keep > n_k) n_keep = n_k;
        }
        const float s = wave_seq_sum_desc(sh.expv, n_keep);
        const unsigned long long last = sh.cand[n_keep - 1];
        const uint32_t last_key = static_cast<uint32_t>(last >> 32);
        int tie = 0;
        if (n_keep < n && static_cast<uint32_t>(sh.cand[n_keep] >> 32) == last_key) tie = static_cast<int>(last & 0xffffffffu);
        const float thr = key_value(last_key), lse_kept = m + logf(s);
        if (a.kept_n && n_keep <= a.kept_cap) {
            for (int q = tid; q < n_keep; q += kWave) {
                const unsigned long long c = sh.cand[q];
                a.kept_idx[r * a.kept_cap + q] = static_cast<int32_t>(c & 0xffffffffu);
                a.kept_x[r * a.kept_cap + q] = key_value(static_cast<uint32_t>(c >> 32));
            }
        }
        if (tid == 0) {
            if (a.kept_n) a.kept_n[r] = n_keep <= a.kept_cap ? n_keep : -1;
            a.thr[r] = thr;
            a.tie[r] = tie;
            a.lse_kept[r] = lse_kept;
            if (a.lse_full) a.lse_full[r] = lse_full;
            if (a.targets && a.logprob) {
                const int64_t tg = a.targets[o * a.ts_outer + i_in * a.ts_inner];
                float lp = -INFINITY, lpf = 0.f;
                if (tg >= 0 && tg < vocab) {
                    const float xt = scale_logit<DT, TEMP>(Row<DT>::load1(row, tg), a.tparam);
                    const bool kept = xt > thr || (xt == thr && tg >= tie);
                    if (kept) lp = xt - lse_kept;
                    lpf = xt - lse_full;
                }
                a.logprob[r] = lp;
                if (a.logprob_full) a.logprob_full[r] = lpf;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// rows whose kept set does not fit the on-chip candidate list (top-p alone over a flat distribution, thousands
// of exact ties, or a very large top_k): the same keep predicate found without a sort, by a radix descent over
// the order keys.  A pass streams the row once and fills a histogram over one digit of the keys that share the
// digits chosen so far: the number of elements per bin, which is what top-k descends by (the largest key with at
// least top_k keys at or above it), and their probability mass per bin, which is what top-p descends by (the
// smallest key whose cumulative mass from below exceeds (1 - p) Z).  A 16-bit logit has 16 significant key bits:
// two digits, so top-k and top-p together take three passes (the first histogram serves both), top-p alone two;
// fp16 adds a three-bit digit, fp32 has four digits.  One more pass over the row and a look at one block of it
// find the first survivor among the elements that tie with the top-p threshold.  The row (at most a few hundred
// KB) comes from cache after the first pass.
//
// Masses are summed as 64-bit fixed-point integers (exp(x - max) * 2^S with S chosen from the row length so that a
// whole row cannot overflow): integer addition is associative, so the LDS atomics that fill the histogram give
// the same sums whatever order they arrive in, and the row's result does not depend on scheduling.  The fixed
// point resolves 2^-45 of the largest element's mass at V = 151936; what it drops is below the rounding of the
// reference's fp32 sums by orders of magnitude, and which of two nearly equal neighbours at the top-p boundary
// falls first may differ from a sorted fp32 running sum, as it may between any two summation orders.
// ---------------------------------------------------------------------------------------------
constexpr int kRadixBins = 256;
constexpr int kRadixCopies = 8;   // histogram copies by lane: logits of one magnitude share their leading digit
constexpr int kTieBlocks = kRadixBins * kRadixCopies;  // index blocks of the tie search (they reuse the count bins)

// digits of an order key from the top, by element type: 16-bit types leave the low key bits constant for a given sign
template <int DT> struct KeyDigits;
template <> struct KeyDigits<NRL_F32> {
    static constexpr int N = 4, LOW = 0;
    __device__ static constexpr int shift(int l) { return 24 - 8 * l; }
    __device__ static constexpr int bits(int) { return 8; }
};
template <> struct KeyDigits<NRL_BF16> {
    static constexpr int N = 2, LOW = 16;
    __device__ static constexpr int shift(int l) { return 24 - 8 * l; }
    __device__ static constexpr int bits(int) { return 8; }
};
template <> struct KeyDigits<NRL_F16> {
    static constexpr int N = 3, LOW = 13;
    __device__ static constexpr int shift(int l) { return l == 2 ? 13 : 24 - 8 * l; }
    __device__ static constexpr int bits(int l) { return l == 2 ? 3 : 8; }
};

struct WideShared {
    unsigned long long mass[kRadixBins * kRadixCopies];
    unsigned int cnt[kRadixBins * kRadixCopies];
    unsigned long long scan64[kSelWaves];
    unsigned int scan32[kSelWaves];
    // what the thread that owns the chosen bin tells the others
    unsigned int pick_bin, pick_cnt;
    unsigned long long pick_a, pick_b;
};

template <typename T> __device__ __forceinline__ T wide_scan_excl(T v, T* shm, T& total) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    T inc = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const T t = __shfl_up(inc, off, kWave);
        if (lane >= off) inc += t;
    }
    __syncthreads();  // the previous scan's readers are done with shm
    if (lane == kWave - 1) shm[wave] = inc;
    __syncthreads();
    T base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kSelWaves; ++w) {
        const T part = shm[w];
        if (w < wave) base += part;
        tot += part;
    }
    total = tot;
    return base + inc - v;
}

// exp(x - m) as a fixed-point integer with fx_shift fraction bits (x <= m, 23 <= fx_shift <= 46); zero below its
// resolution.  Without branches: the 24-bit significand is placed where the value 1.0 belongs and moved down by
// the exponent's distance from 1.0's.
__device__ __forceinline__ unsigned long long wide_mass(float x, float m, int fx_shift) {
    const uint32_t b = __float_as_uint(fast_exp2((x - m) * kLog2e)) & 0x7fffffffu;
    const int ex = static_cast<int>(b >> 23);
    const unsigned long long top = static_cast<unsigned long long>((b & 0x7fffffu) | 0x800000u) << (fx_shift - 23);
    int down = 127 - ex;              // 0 for 1.0; 127 for zero and subnormals (flushed); negative never for x <= m
    down = down < 0 ? 0 : down > 63 ? 63 : down;
    return ex == 255 ? 0ull : top >> down;   // (a NaN logit weighs nothing)
}

template <int DT, int TEMP> struct WideRow {
    const char* row;
    const u32x4* xv;
    int64_t vocab, head, nvec, tail0;
    float tparam;
    // f(scaled logit, vocabulary index) for every element of the row, each exactly once
    template <typename F> __device__ __forceinline__ void for_each(F f) const {
        constexpr int EPV = Row<DT>::EPV;
        constexpr int kLoads = 8;  // vector loads in flight per thread: a pass is bound by their latency otherwise
        const int tid = threadIdx.x;
        int64_t vi = tid;
        for (; vi + (kLoads - 1) * kSelBlock < nvec; vi += kLoads * kSelBlock) {
            u32x4 q[kLoads];
#pragma unroll
            for (int u = 0; u < kLoads; ++u) q[u] = xv[vi + u * kSelBlock];
#pragma unroll
            for (int u = 0; u < kLoads; ++u) {
                float t[EPV];
                Row<DT>::decode(q[u], t);
#pragma unroll
                for (int k = 0; k < EPV; ++k) f(scale_logit<DT, TEMP>(t[k], tparam), head + (vi + u * kSelBlock) * EPV + k);
            }
        }
        for (; vi < nvec; vi += kSelBlock) {
            float t[EPV];
            Row<DT>::decode(xv[vi], t);
#pragma unroll
            for (int k = 0; k < EPV; ++k) f(scale_logit<DT, TEMP>(t[k], tparam), head + vi * EPV + k);
        }
        if (tid < head) f(scale_logit<DT, TEMP>(Row<DT>::load1(row, tid), tparam), static_cast<int64_t>(tid));
        if (tail0 + tid < vocab) f(scale_logit<DT, TEMP>(Row<DT>::load1(row, tail0 + tid), tparam), tail0 + tid);
    }
};

// One histogram pass: bin = digit `level` of the keys whose higher digits equal `prefix` (every key at level 0).
// Thread b returns the mass of such elements in bin b and, with CNT, their number (0 otherwise: the top-p descent
// needs counts at its last digit only, and every atomic less shortens the pass).
template <int DT, int TEMP, bool CNT>
__device__ __forceinline__ void wide_hist_pass(const WideRow<DT, TEMP>& w, WideShared& sh, float m, int fx_shift, int level,
                                               uint32_t prefix, unsigned int& my_cnt, unsigned long long& my_mass) {
    const int tid = threadIdx.x;
    const int shift = KeyDigits<DT>::shift(level), bits = KeyDigits<DT>::bits(level);
    const uint32_t mask = (1u << bits) - 1u;
    __syncthreads();  // whoever still reads the bins of the pass before
    for (int i = tid; i < kRadixBins * kRadixCopies; i += kSelBlock) { sh.mass[i] = 0ull; sh.cnt[i] = 0u; }
    __syncthreads();
    const int copy = tid & (kRadixCopies - 1);
    if (level == 0) {
        w.for_each([&](float x, int64_t) {
            const int slot = static_cast<int>((order_key(x) >> shift) & mask) * kRadixCopies + copy;
            if (CNT) atomicAdd(&sh.cnt[slot], 1u);
            atomicAdd(&sh.mass[slot], wide_mass(x, m, fx_shift));
        });
    } else {
        w.for_each([&](float x, int64_t) {
            const uint32_t key = order_key(x);
            if ((key >> (shift + bits)) == prefix) {
                const int slot = static_cast<int>((key >> shift) & mask) * kRadixCopies + copy;
                if (CNT) atomicAdd(&sh.cnt[slot], 1u);
                atomicAdd(&sh.mass[slot], wide_mass(x, m, fx_shift));
            }
        });
    }
    __syncthreads();
    my_cnt = 0u;
    my_mass = 0ull;
#pragma unroll
    for (int q = 0; q < kRadixCopies; ++q) {
        my_cnt += sh.cnt[tid * kRadixCopies + q];
        my_mass += sh.mass[tid * kRadixCopies + q];
    }
}

template <int DT, int TEMP>
__global__ __launch_bounds__(kSelBlock) void topk_topp_wide_kernel(SelArgs a, int64_t n_rows) {
    static_assert(kRadixBins == kSelBlock, "one histogram bin per thread");
    __shared__ WideShared sh;
    using KD = KeyDigits<DT>;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const bool use_p = a.top_p < 1.0f;
    {
        // the usual case is that no row of this workgroup is marked: look at all of them at once and leave
        bool mine = false;
        for (int64_t r = blockIdx.x + static_cast<int64_t>(tid) * gridDim.x; r < n_rows; r += static_cast<int64_t>(kSelBlock) * gridDim.x)
            mine |= a.tie[r] == kTieUnresolved;
        if (!__syncthreads_or(mine)) return;
    }
    int clog2 = 0;
    while ((int64_t{1} << clog2) < a.vocab) ++clog2;
    const int fx_shift = 63 - clog2 < 46 ? 63 - clog2 : 46;  // a row of `vocab` largest elements still fits 63 bits
    for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) {
        if (a.tie[r] != kTieUnresolved) continue;  // the same word for every thread of the workgroup
        const int64_t o = r / a.n_inner, i_in = r - o * a.n_inner;
        WideRow<DT, TEMP> w;
        w.row = static_cast<const char*>(a.logits) + (o * a.stride_outer + i_in * a.stride_inner) * Row<DT>::BYTES;
        w.vocab = a.vocab;
        w.head = sel_row_head<DT>(w.row, w.vocab);
        w.nvec = (w.vocab - w.head) / Row<DT>::EPV;
        w.tail0 = w.head + w.nvec * Row<DT>::EPV;
        w.xv = reinterpret_cast<const u32x4*>(w.row + w.head * Row<DT>::BYTES);
        w.tparam = a.tparam;
        const float m = a.thr[r];  // the row's largest (scaled) logit, left here by the kernel that marked the row
        const bool use_k = a.top_k > 0 && a.top_k < w.vocab;

        // ---- first digit, every element: serves the top-k and the top-p descent alike ----
        unsigned int hc[KD::N];         // this thread's bin along the top-k descent (or just level 0), per level
        unsigned long long hm[KD::N];
        uint32_t hprefix[KD::N];
        int h_levels = 1;
        hprefix[0] = 0u;
        if (use_k) wide_hist_pass<DT, TEMP, true>(w, sh, m, fx_shift, 0, 0u, hc[0], hm[0]);
        else wide_hist_pass<DT, TEMP, KD::N == 1>(w, sh, m, fx_shift, 0, 0u, hc[0], hm[0]);
        unsigned long long total_mass = 0ull;
        wide_scan_excl(hm[0], sh.scan64, total_mass);

        // ---- top-k: the largest key with at least top_k keys at or above it (ties at that key are all kept) ----
        uint32_t k_key = 0u;
        unsigned long long mass_below_k = 0ull;
        unsigned int cnt_at_k = 0u;
        if (use_k) {
            unsigned int need = static_cast<unsigned int>(a.top_k);
            uint32_t prefix = 0u;
#pragma unroll
            for (int l = 0; l < KD::N; ++l) {
                if (l > 0) {
                    hprefix[l] = prefix;
                    wide_hist_pass<DT, TEMP, true>(w, sh, m, fx_shift, l, prefix, hc[l], hm[l]);
                    h_levels = l + 1;
                }
                unsigned int tot_c = 0u;
                unsigned long long tot_m = 0ull;
                const unsigned int excl_c = wide_scan_excl(hc[l], sh.scan32, tot_c);
                const unsigned long long excl_m = wide_scan_excl(hm[l], sh.scan64, tot_m);
                const unsigned int at_or_above = tot_c - excl_c, above = at_or_above - hc[l];
                if (at_or_above >= need && above < need) {
                    sh.pick_bin = static_cast<unsigned int>(tid);
                    sh.pick_cnt = hc[l];
                    sh.pick_a = need - above;
                    sh.pick_b = excl_m;
                }
                __syncthreads();
                prefix = (prefix << KD::bits(l)) | sh.pick_bin;
                need = static_cast<unsigned int>(sh.pick_a);
                mass_below_k += sh.pick_b;
                cnt_at_k = sh.pick_cnt;
                __syncthreads();  // everyone has read the pick
            }
            k_key = prefix << KD::LOW;
            if (KD::LOW > 0 && !(k_key >> 31)) k_key |= (1u << KD::LOW) - 1u;  // a negative value's low key bits are ones
        }
        const unsigned long long z = total_mass - mass_below_k;  // mass of the top-k survivors

        uint32_t thr_key = k_key;
        int32_t tie = 0;
        unsigned long long kept_mass = z;
        if (use_p) {
            // ascending cumulative probability over the survivors; elements fall while it stays <= (1 - p) Z.  Counted
            // over the whole row that is: mass below the key <= (1 - p) Z + mass below the top-k threshold.
            const double target_d = static_cast<double>(1.0f - a.top_p) * static_cast<double>(z);
            const unsigned long long target = target_d <= 0.0 ? 0ull : static_cast<unsigned long long>(target_d);
            unsigned long long room = target + mass_below_k;  // what may still lie below the digit being chosen
            unsigned long long below_all = 0ull;
            unsigned int n_eq = 0u;
            uint32_t prefix = 0u;
#pragma unroll
            for (int l = 0; l < KD::N; ++l) {
                unsigned int bc = hc[l];
                unsigned long long bm = hm[l];
                if (l >= h_levels || hprefix[l] != prefix) {
                    if (l == KD::N - 1) wide_hist_pass<DT, TEMP, true>(w, sh, m, fx_shift, l, prefix, bc, bm);
                    else wide_hist_pass<DT, TEMP, false>(w, sh, m, fx_shift, l, prefix, bc, bm);
                }
                unsigned long long tot_m = 0ull;
                const unsigned long long excl_m = wide_scan_excl(bm, sh.scan64, tot_m);
                // the bin in which the cumulative mass first exceeds the room; if it never does (top_p -> 0), the
                // highest bin with any mass, which holds the largest element: that one always survives
                const bool crossing = tot_m > room ? (excl_m + bm > room && excl_m <= room)
                                                   : (bm > 0ull && tot_m - excl_m - bm == 0ull);
                if (crossing) {
                    sh.pick_bin = static_cast<unsigned int>(tid);
                    sh.pick_cnt = bc;
                    sh.pick_a = room - excl_m;
                    sh.pick_b = excl_m;
                }
                __syncthreads();
                prefix = (prefix << KD::bits(l)) | sh.pick_bin;
                room = sh.pick_a;
                below_all += sh.pick_b;
                n_eq = sh.pick_cnt;
                __syncthreads();
            }
            uint32_t c = prefix << KD::LOW;
            if (KD::LOW > 0 && !(c >> 31)) c |= (1u << KD::LOW) - 1u;
            unsigned long long below = 0ull;  // mass of the survivors strictly below the threshold
            if (c <= k_key) { c = k_key; if (use_k) n_eq = cnt_at_k; }
            else below = below_all - mass_below_k;
            thr_key = c;
            // how many of the elements equal to the threshold fall too (the ones with the smallest indices)
            const unsigned long long e_thr = wide_mass(key_value(c), m, fx_shift);
            unsigned long long drop = 0ull;
            if (e_thr > 0ull && n_eq > 1u && target >= below) {
                drop = (target - below) / e_thr;
                if (drop > n_eq - 1u) drop = n_eq - 1u;
            }
            if (drop > 0ull) {
                // index of the first survivor among the equal elements, the one with `drop` equal elements before it:
                // equal elements counted per block of indices, then one look at the block that holds it
                int ishift = clog2 - 11;
                if (ishift < 0) ishift = 0;
                __syncthreads();
                for (int i = tid; i < kTieBlocks; i += kSelBlock) sh.cnt[i] = 0u;
                __syncthreads();
                w.for_each([&](float x, int64_t j) {
                    if (order_key(x) == c) atomicAdd(&sh.cnt[j >> ishift], 1u);
                });
                __syncthreads();
                unsigned int mine8[kRadixCopies], sum8 = 0u;
#pragma unroll
                for (int q = 0; q < kRadixCopies; ++q) { mine8[q] = sh.cnt[tid * kRadixCopies + q]; sum8 += mine8[q]; }
                unsigned int tot_eq = 0u;
                unsigned int before = wide_scan_excl(sum8, sh.scan32, tot_eq);
                if (before <= drop && drop < before + sum8) {
#pragma unroll
                    for (int q = 0; q < kRadixCopies; ++q) {
                        if (before <= drop && drop < before + mine8[q]) {
                            sh.pick_bin = static_cast<unsigned int>(tid * kRadixCopies + q);
                            sh.pick_cnt = static_cast<unsigned int>(drop) - before;
                        }
                        before += mine8[q];
                    }
                }
                __syncthreads();
                const int64_t first = static_cast<int64_t>(sh.pick_bin) << ishift;
                int64_t stop = first + (int64_t{1} << ishift);
                if (stop > w.vocab) stop = w.vocab;
                unsigned int seen = 0u;
                const unsigned int want = sh.pick_cnt;
                for (int64_t j0 = first; j0 < stop; j0 += kSelBlock) {
                    const int64_t j = j0 + tid;
                    const bool eq = j < stop && order_key(scale_logit<DT, TEMP>(Row<DT>::load1(w.row, j), a.tparam)) == c;
                    const unsigned long long bal = __ballot(eq);
                    const unsigned int in_wave = static_cast<unsigned int>(__popcll(bal & ((1ull << lane) - 1ull)));
                    __syncthreads();
                    if (lane == 0) sh.scan32[wave] = static_cast<unsigned int>(__popcll(bal));
                    __syncthreads();
                    unsigned int ahead = seen, chunk = 0u;
#pragma unroll
                    for (int q = 0; q < kSelWaves; ++q) {
                        if (q < wave) ahead += sh.scan32[q];
                        chunk += sh.scan32[q];
                    }
                    if (eq && ahead + in_wave == want) sh.pick_a = static_cast<unsigned long long>(j);
                    seen += chunk;
                }
                __syncthreads();
                tie = static_cast<int32_t>(sh.pick_a);
            }
            kept_mass = z - below - drop * e_thr;
            if (kept_mass == 0ull || kept_mass > z) kept_mass = e_thr;
        }
        const float thr = key_value(thr_key);
        const float unit = __uint_as_float(static_cast<uint32_t>(127 - fx_shift) << 23);  // 2^-fx_shift
        const float lse_kept = m + logf(static_cast<float>(static_cast<double>(kept_mass) * static_cast<double>(unit)));
        const float lse_full = m + logf(static_cast<float>(static_cast<double>(total_mass) * static_cast<double>(unit)));
        __syncthreads();      // every thread has read thr[r] (the row maximum) and tie[r] == unresolved before they are replaced
        if (tid == 0) {
            a.thr[r] = thr;
            a.lse_kept[r] = lse_kept;
            if (a.lse_full) a.lse_full[r] = lse_full;
            if (a.targets && a.logprob) {
                const int64_t tg = a.targets[o * a.ts_outer + i_in * a.ts_inner];
                float lp = -INFINITY, lpf = 0.f;
                if (tg >= 0 && tg < w.vocab) {
                    const float xt = scale_logit<DT, TEMP>(Row<DT>::load1(w.row, tg), a.tparam);
                    const bool kept = xt > thr || (xt == thr && tg >= tie);
                    if (kept) lp = xt - lse_kept;
                    lpf = xt - lse_full;
                }
                a.logprob[r] = lp;
                if (a.logprob_full) a.logprob_full[r] = lpf;
            }
            a.tie[r] = tie;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// backward / materialisation: one streaming pass with the saved keep predicate
// ---------------------------------------------------------------------------------------------
struct SelBwdArgs {
    const void* logits;
    int64_t n_inner, vocab, stride_outer, stride_inner;
    const int64_t* targets;
    int64_t ts_outer, ts_inner;
    float tparam;
    const float* thr;
    const int32_t* tie;
    const float* lse_kept;
    const float* grad;
    int64_t gs_outer, gs_inner;
    void* out;  // dlogits, or filtered logits
    int64_t d_n_inner, ds_outer, ds_inner;
    uint8_t* keep_out;  // [rows, vocab] or NULL (filter mode)
    const int32_t* kept_n;    // the forward's record of the kept sets (see SelArgs), or NULL
    const int32_t* kept_idx;
    const float* kept_x;
    int kept_cap;
    int prefilled;  // the record is in use: the whole gradient buffer was zero-filled before this launch, rows on record only add their entries
};

// MODE 0: gradient, MODE 1: filtered logits (-inf outside the kept set) + keep mask
template <int DT, int TEMP, int MODE>
__device__ __forceinline__ void topk_topp_stream_row(const SelBwdArgs& a, int64_t r) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const int64_t o = r / a.d_n_inner, i_in = r - o * a.d_n_inner;
    char* out = static_cast<char*>(a.out) + (o * a.ds_outer + i_in * a.ds_inner) * Row<DT>::BYTES;
    const int64_t vocab = a.vocab;
    float g = 0.f;
    if (MODE == 0 && i_in < a.n_inner) g = a.grad[o * a.gs_outer + i_in * a.gs_inner];
    // With the forward's record of the kept set the gradient row is zeros plus the few kept entries, written
    // without reading the logits again.
    int n_rec = -1;
    if (MODE == 0 && g != 0.f && a.prefilled) {
        n_rec = a.kept_n[o * a.n_inner + i_in];
        if (n_rec > a.kept_cap) n_rec = -1;  // not a count the forward writes: stream the row instead
    }
    if (MODE == 0 && a.prefilled && (g == 0.f || n_rec >= 0)) {
        // the zeros are there already (an earlier launch on the stream): only the kept entries are written
        const int64_t rec = (o * a.n_inner + i_in) * a.kept_cap;
        if (n_rec > 0) {
            const float lse_r = a.lse_kept[o * a.n_inner + i_in];
            const int64_t tg_r = a.targets[o * a.ts_outer + i_in * a.ts_inner];
            for (int q = tid; q < n_rec; q += kSelBlock) {
                const int64_t idx = a.kept_idx[rec + q];
                if (static_cast<uint64_t>(idx) >= static_cast<uint64_t>(vocab)) continue;
                float d = ((idx == tg_r ? 1.f : 0.f) - fast_exp2((a.kept_x[rec + q] - lse_r) * kLog2e)) * g;
                if constexpr (TEMP == 1) d = __fdiv_rn(Row<DT>::round_self(d), a.tparam);
                if constexpr (TEMP == 2) d = Row<DT>::round_self(d) * a.tparam;
                Row<DT>::store1(out, idx, d);
            }
        }
        return;
    }
    if (MODE == 0 && g == 0.f) {  // dropped position or masked token: the gradient row is exactly zero
        const int64_t zh = sel_row_head<DT>(out, vocab);
        const int64_t zn = (vocab - zh) / EPV;
        u32x4* zv = reinterpret_cast<u32x4*>(out + zh * Row<DT>::BYTES);
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int64_t v = tid; v < zn; v += kSelBlock) zv[v] = z;
        if (tid < zh) Row<DT>::store1(out, tid, 0.f);
        if (zh + zn * EPV + tid < vocab) Row<DT>::store1(out, zh + zn * EPV + tid, 0.f);
        return;
    }
    const int64_t rr = o * a.n_inner + i_in;
    const char* row = static_cast<const char*>(a.logits) + (o * a.stride_outer + i_in * a.stride_inner) * Row<DT>::BYTES;
    const float thr = a.thr[rr], lse = a.lse_kept[rr];
    const int64_t tie = a.tie[rr];
    int64_t tg = -1;
    if (MODE == 0) tg = a.targets[o * a.ts_outer + i_in * a.ts_inner];
    uint8_t* keep_row = (MODE == 1 && a.keep_out) ? a.keep_out + rr * vocab : nullptr;

    auto elem = [&](float x_raw, int64_t idx, bool& keep) -> float {
        const float x = scale_logit<DT, TEMP>(x_raw, a.tparam);
        keep = x > thr || (x == thr && idx >= tie);
        if (MODE == 1) return keep ? x : -INFINITY;
        if (!keep) return 0.f;
        float d = ((idx == tg ? 1.f : 0.f) - fast_exp2((x - lse) * kLog2e)) * g;
        if constexpr (TEMP == 1) d = __fdiv_rn(Row<DT>::round_self(d), a.tparam);
        if constexpr (TEMP == 2) d = Row<DT>::round_self(d) * a.tparam;
        return d;
    };

    const int64_t head = sel_row_head<DT>(row, vocab);
    if (sel_row_head<DT>(out, vocab) != head) {
        for (int64_t e = tid; e < vocab; e += kSelBlock) {
            bool keep;
            Row<DT>::store1(out, e, elem(Row<DT>::load1(row, e), e, keep));
            if (keep_row) keep_row[e] = keep ? 1 : 0;
        }
        return;
    }
    const int64_t nvec = (vocab - head) / EPV;
    const int64_t tail0 = head + nvec * EPV;
    const u32x4* xv = reinterpret_cast<const u32x4*>(row + head * Row<DT>::BYTES);
    u32x4* ov = reinterpret_cast<u32x4*>(out + head * Row<DT>::BYTES);
    // the keep flags of a vector leave as one EPV-byte store where the mask row allows it (one byte store per element
    // made the filter 27 % slower)
    using MaskWord = typename std::conditional<EPV == 8, uint64_t, uint32_t>::type;
    static_assert(sizeof(MaskWord) == EPV, "one mask byte per element of a vector");
    const bool mask_words = keep_row && ((reinterpret_cast<uintptr_t>(keep_row) + head) % EPV) == 0;
    for (int64_t vi = tid; vi < nvec; vi += kSelBlock) {
        float t[EPV];
        Row<DT>::decode(__builtin_nontemporal_load(xv + vi), t);
        MaskWord bits = 0;
#pragma unroll
        for (int k = 0; k < EPV; ++k) {
            bool keep;
            const int64_t idx = head + vi * EPV + k;
            t[k] = elem(t[k], idx, keep);
            bits |= static_cast<MaskWord>(keep ? 1 : 0) << (8 * k);
            if (keep_row && !mask_words) keep_row[idx] = keep ? 1 : 0;
        }
        if (mask_words) *reinterpret_cast<MaskWord*>(keep_row + head + vi * EPV) = bits;
        __builtin_nontemporal_store(Row<DT>::encode(t), ov + vi);
    }
    for (int w = 0; w < 2; ++w) {
        const int64_t e = w == 0 ? (tid < head ? tid : -1) : (tail0 + tid < vocab ? tail0 + tid : -1);
        if (e < 0) continue;
        bool keep;
        Row<DT>::store1(out, e, elem(Row<DT>::load1(row, e), e, keep));
        if (keep_row) keep_row[e] = keep ? 1 : 0;
    }
}

// Zero fill of a contiguous buffer by one workgroup per compute unit in 256 KiB spans: 6.0 TB/s, as a memset, where
// one workgroup per row reaches 5.5.
constexpr int kFillGrid = 256;
constexpr int64_t kFillSpan = 256 * 1024;
__global__ __launch_bounds__(256) void fill_zero_flat_kernel(char* out, int64_t total_bytes) {
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int64_t s0 = static_cast<int64_t>(blockIdx.x) * kFillSpan; s0 < total_bytes; s0 += static_cast<int64_t>(gridDim.x) * kFillSpan) {
        u32x4* zv = reinterpret_cast<u32x4*>(out + s0);
        const int64_t left = total_bytes - s0;
        const int64_t nv = (left < kFillSpan ? left : kFillSpan) / 16;
        for (int64_t v = threadIdx.x; v < nv; v += 256) zv[v] = z;
        if (left < kFillSpan && threadIdx.x < (left & 15)) out[s0 + nv * 16 + threadIdx.x] = 0;
    }
}

// One workgroup per row (a fixed set of 512 workgroups walking the rows, which fills memory 10 % faster when it does
// nothing else, measured no gain here: with few workgroups per compute unit the record staging of a row is exposed).
template <int DT, int TEMP, int MODE>
__global__ __launch_bounds__(kSelBlock) void topk_topp_stream_kernel(SelBwdArgs a, int64_t n_rows) {
    for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) topk_topp_stream_row<DT, TEMP, MODE>(a, r);
}

static int temp_code3(float temperature, int mode, float* tparam) {
    if (temperature == 1.0f) { *tparam = 1.f; return 0; }
    if (mode == NRL_TEMP_DIV) { *tparam = temperature; return 1; }
    *tparam = 1.0f / temperature;
    return 2;
}

static int check_sel_rows(const nrl_rows* r, bool need_targets) {
    if (!r) return fail(NRL_E_INVALID, "rows is NULL");
    if (r->dtype != NRL_F32 && r->dtype != NRL_BF16 && r->dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown logits dtype %d", r->dtype);
    if (r->n_outer < 0 || r->n_inner < 0 || r->vocab <= 0) return fail(NRL_E_INVALID, "bad shape");
    if (r->vocab >= (1ll << 31)) return fail(NRL_E_INVALID, "vocabulary too large");
    if (r->n_outer * r->n_inner > 0 && (!r->logits || (need_targets && !r->targets))) return fail(NRL_E_INVALID, "null logits or targets");
    if (r->vocab_start != 0 || r->vocab_end != r->vocab) return fail(NRL_E_UNSUPPORTED, "top-k/top-p needs the full vocabulary on this GPU");
    if (!(r->temperature > 0.f)) return fail(NRL_E_INVALID, "temperature must be positive");
    if (r->n_outer * r->n_inner >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    return NRL_OK;
}

#define NRL_SEL_DISPATCH(DT_, TC_, ...)                                                     \
    switch ((DT_) * 3 + (TC_)) {                                                            \
        case NRL_F32 * 3 + 0: { constexpr int DT = NRL_F32, TEMP = 0; __VA_ARGS__; break; }  \
        case NRL_F32 * 3 + 1: { constexpr int DT = NRL_F32, TEMP = 1; __VA_ARGS__; break; }  \
        case NRL_F32 * 3 + 2: { constexpr int DT = NRL_F32, TEMP = 2; __VA_ARGS__; break; }  \
        case NRL_BF16 * 3 + 0: { constexpr int DT = NRL_BF16, TEMP = 0; __VA_ARGS__; break; } \
        case NRL_BF16 * 3 + 1: { constexpr int DT = NRL_BF16, TEMP = 1; __VA_ARGS__; break; } \
        case NRL_BF16 * 3 + 2: { constexpr int DT = NRL_BF16, TEMP = 2; __VA_ARGS__; break; } \
        case NRL_F16 * 3 + 0: { constexpr int DT = NRL_F16, TEMP = 0; __VA_ARGS__; break; }  \
        case NRL_F16 * 3 + 1: { constexpr int DT = NRL_F16, TEMP = 1; __VA_ARGS__; break; }  \
        default: { constexpr int DT = NRL_F16, TEMP = 2; __VA_ARGS__; break; }              \
    }

}  // namespace nrl

using namespace nrl;

extern "C" int nrl_topk_topp_logprob_fwd(const nrl_rows* rows, int64_t top_k, float top_p, float* logprob_out,
                                         float* thr_out, int32_t* tie_out, float* lse_kept_out,
                                         float* logprob_unfiltered_out, float* lse_full_out, int32_t* kept_count_out,
                                         int32_t* kept_index_out, float* kept_value_out, int64_t kept_capacity,
                                         void* stream) {
    if (int e = check_sel_rows(rows, logprob_out != nullptr)) return e;
    const bool use_k = top_k > 0, use_p = top_p < 1.0f;
    if (!use_k && !use_p) return fail(NRL_E_INVALID, "neither top-k nor top-p is active");
    if (use_p && !(top_p > 0.f)) return fail(NRL_E_INVALID, "top_p must be in (0, 1]");
    const int64_t n = rows->n_outer * rows->n_inner;
    if (n == 0) return NRL_OK;
    if (!thr_out || !tie_out || !lse_kept_out) return fail(NRL_E_INVALID, "null state output");
    if (kept_count_out && (!kept_index_out || !kept_value_out || kept_capacity < 1 || kept_capacity > kCapSmall))
        return fail(NRL_E_INVALID, "kept-set record: index and value outputs and a capacity in [1, %d] are needed", kCapSmall);
    SelArgs a;
    a.kept_n = kept_count_out; a.kept_idx = kept_index_out; a.kept_x = kept_value_out; a.kept_cap = static_cast<int>(kept_capacity);
    a.logits = rows->logits; a.n_inner = rows->n_inner; a.vocab = rows->vocab;
    a.stride_outer = rows->stride_outer; a.stride_inner = rows->stride_inner;
    a.targets = rows->targets; a.ts_outer = rows->tgt_stride_outer; a.ts_inner = rows->tgt_stride_inner;
    a.top_k = use_k ? static_cast<int>(top_k > (1ll << 30) ? (1ll << 30) : top_k) : 0;
    a.top_p = use_p ? top_p : 1.0f;
    a.logprob = logprob_out; a.thr = thr_out; a.tie = tie_out; a.lse_kept = lse_kept_out;
    a.logprob_full = logprob_unfiltered_out; a.lse_full = lse_full_out;
    const int tc = temp_code3(rows->temperature, rows->temp_mode, &a.tparam);
    const bool full = !use_k || logprob_unfiltered_out != nullptr || lse_full_out != nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool small = use_k && a.top_k <= kSmallTopK;
    if (!use_k) {
        NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_fwd_kernel<DT, TEMP, true, kCap, true><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a));
    } else if (full && small) {
        NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_fwd_kernel<DT, TEMP, true, kCapSmall><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a));
    } else if (full) {
        NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_fwd_kernel<DT, TEMP, true, kCap><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a));
    } else if (small) {
        NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_fwd_kernel<DT, TEMP, false, kCapSmall><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a));
    } else {
        NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_fwd_kernel<DT, TEMP, false, kCap><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a));
    }
    if (int e = check_launch("topk_topp_logprob_fwd")) return e;
    // rows the candidate list could not hold are finished here; with none, every workgroup leaves after
    // reading its rows' markers
    const unsigned grid = static_cast<unsigned>(n < kWideGrid ? n : kWideGrid);
    NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_wide_kernel<DT, TEMP><<<dim3(grid), dim3(kSelBlock), 0, s>>>(a, n));
    return check_launch("topk_topp_logprob_fwd (wide rows)");
}

extern "C" int nrl_topk_topp_logprob_bwd(const nrl_rows* rows, const float* thr, const int32_t* tie,
                                         const float* lse_kept, const float* grad, int64_t grad_stride_outer,
                                         int64_t grad_stride_inner, const int32_t* kept_count, const int32_t* kept_index,
                                         const float* kept_value, int64_t kept_capacity, void* dlogits, int64_t d_n_inner,
                                         int64_t d_stride_outer, int64_t d_stride_inner, void* stream) {
    if (int e = check_sel_rows(rows, true)) return e;
    if (d_n_inner < rows->n_inner) return fail(NRL_E_INVALID, "d_n_inner < n_inner");
    const int64_t n = rows->n_outer * d_n_inner;
    if (n == 0) return NRL_OK;
    if (n >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    if (!dlogits || (rows->n_outer * rows->n_inner > 0 && (!thr || !tie || !lse_kept || !grad))) return fail(NRL_E_INVALID, "null argument");
    SelBwdArgs a;
    a.logits = rows->logits; a.n_inner = rows->n_inner; a.vocab = rows->vocab;
    a.stride_outer = rows->stride_outer; a.stride_inner = rows->stride_inner;
    a.targets = rows->targets; a.ts_outer = rows->tgt_stride_outer; a.ts_inner = rows->tgt_stride_inner;
    a.thr = thr; a.tie = tie; a.lse_kept = lse_kept; a.grad = grad;
    a.gs_outer = grad_stride_outer; a.gs_inner = grad_stride_inner;
    a.out = dlogits; a.d_n_inner = d_n_inner; a.ds_outer = d_stride_outer; a.ds_inner = d_stride_inner;
    a.keep_out = nullptr;
    if (kept_count && (!kept_index || !kept_value || kept_capacity < 1)) return fail(NRL_E_INVALID, "incomplete kept-set record");
    a.kept_n = kept_count; a.kept_idx = kept_index; a.kept_x = kept_value; a.kept_cap = static_cast<int>(kept_capacity);
    const int tc = temp_code3(rows->temperature, rows->temp_mode, &a.tparam);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // With the kept sets on record nearly every row is zeros plus a few entries.  A gradient buffer that is one
    // contiguous block is then zero-filled flat, which writes faster than row by row, and the row launch only adds
    // the entries (and streams the rows that are not on record).  For a strided buffer the record is left unused.
    const int64_t elt = rows->dtype == NRL_F32 ? 4 : 2;
    a.prefilled = kept_count && d_stride_inner == rows->vocab && d_stride_outer == d_n_inner * rows->vocab &&
                  (reinterpret_cast<uintptr_t>(dlogits) & 15) == 0;
    if (a.prefilled && rows->logits && rows->n_outer * rows->n_inner > 0) {
        // A gradient written over the logits (allowed, as for nrl_logprob_bwd) must not be cleared first: rows that
        // are not on record still stream from the logits.  Such a call takes the row-by-row path, which reads a
        // vector before it overwrites it.
        const uintptr_t d0 = reinterpret_cast<uintptr_t>(dlogits), d1 = d0 + static_cast<uintptr_t>(n * rows->vocab * elt);
        const uintptr_t l0 = reinterpret_cast<uintptr_t>(rows->logits);
        const int64_t so = rows->stride_outer < 0 ? -rows->stride_outer : rows->stride_outer;
        const int64_t si = rows->stride_inner < 0 ? -rows->stride_inner : rows->stride_inner;
        const uintptr_t l1 = l0 + static_cast<uintptr_t>(((rows->n_outer - 1) * so + (rows->n_inner - 1) * si + rows->vocab) * elt);
        if (d0 < l1 && l0 < d1) a.prefilled = 0;
    }
    if (a.prefilled) fill_zero_flat_kernel<<<dim3(kFillGrid), dim3(256), 0, s>>>(static_cast<char*>(dlogits), n * rows->vocab * elt);
    NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_stream_kernel<DT, TEMP, 0><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a, n));
    return check_launch("topk_topp_logprob_bwd");
}

extern "C" int nrl_topk_topp_filter(const nrl_rows* rows, const float* thr, const int32_t* tie, void* filtered_out,
                                    int64_t f_stride_outer, int64_t f_stride_inner, uint8_t* keep_out, void* stream) {
    if (int e = check_sel_rows(rows, false)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (n == 0) return NRL_OK;
    if (!thr || !tie || !filtered_out) return fail(NRL_E_INVALID, "null argument");
    SelBwdArgs a;
    a.logits = rows->logits; a.n_inner = rows->n_inner; a.vocab = rows->vocab;
    a.stride_outer = rows->stride_outer; a.stride_inner = rows->stride_inner;
    a.targets = nullptr; a.ts_outer = 0; a.ts_inner = 0;
    a.thr = thr; a.tie = tie; a.lse_kept = thr; a.grad = nullptr; a.gs_outer = 0; a.gs_inner = 0;
    a.out = filtered_out; a.d_n_inner = rows->n_inner; a.ds_outer = f_stride_outer; a.ds_inner = f_stride_inner;
    a.keep_out = keep_out;
    a.kept_n = nullptr; a.kept_idx = nullptr; a.kept_x = nullptr; a.kept_cap = 0; a.prefilled = 0;
    const int tc = temp_code3(rows->temperature, rows->temp_mode, &a.tparam);
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_SEL_DISPATCH(rows->dtype, tc, topk_topp_stream_kernel<DT, TEMP, 1><<<dim3((unsigned)n), dim3(kSelBlock), 0, s>>>(a, n));
    return check_launch("topk_topp_filter");
}

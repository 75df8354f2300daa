// Full-vocabulary reductions that distillation losses need, on the same one-pass-per-row streaming core as
// the token logprob kernels (one 256-thread workgroup per row, 16-byte loads, online rescaling):
//   * sum_v p_v log p_v (the negative entropy) and its gradient,
//   * log-probabilities gathered at K given vocabulary indices per row and their gradient,
//   * soft-target cross entropy H(p_teacher, q_student) of two logit tensors and its gradient.
// Rows whose start is not 16-byte aligned (or whose length is not a whole number of vectors) take an
// element-wise path; nothing is ever materialised at [rows, V] in fp32.

#include <float.h>
#include <math.h>

#include "common.hpp"

namespace nrl {

constexpr int kDBlock = 256;
constexpr int kDWaves = kDBlock / kWave;
constexpr int kDUnroll = 4;

struct RowsView {
    const void* p;
    int64_t n_inner, vocab, stride_outer, stride_inner;
};

template <int DT> __device__ __forceinline__ const char* row_ptr(const RowsView& v, int64_t r) {
    const int64_t o = r / v.n_inner, i = r - o * v.n_inner;
    return static_cast<const char*>(v.p) + (o * v.stride_outer + i * v.stride_inner) * Row<DT>::BYTES;
}

template <int DT> __device__ __forceinline__ bool vec_ok(const void* row, int64_t vocab) {
    return (reinterpret_cast<uintptr_t>(row) & 15) == 0 && vocab % Row<DT>::EPV == 0;
}

// fv(values of one 16-byte vector) / f1(one element) over the row, each thread taking a strided share
template <int DT, class FV, class F1> __device__ __forceinline__ void row_for_each_vec(const void* row, int64_t vocab, FV fv, F1 f1) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    if (!vec_ok<DT>(row, vocab)) {
        for (int64_t i = tid; i < vocab; i += kDBlock) f1(Row<DT>::load1(row, i));
        return;
    }
    const u32x4* xv = static_cast<const u32x4*>(row);
    const int64_t nvec = vocab / EPV;
    int64_t base = 0;
    for (; base + kDUnroll * kDBlock <= nvec; base += kDUnroll * kDBlock) {
        u32x4 q[kDUnroll];
#pragma unroll
        for (int u = 0; u < kDUnroll; ++u) q[u] = __builtin_nontemporal_load(xv + base + u * kDBlock + tid);
#pragma unroll
        for (int u = 0; u < kDUnroll; ++u) {
            float t[EPV];
            Row<DT>::decode(q[u], t);
            fv(t);
        }
    }
    for (int64_t vi = base + tid; vi < nvec; vi += kDBlock) {
        float t[EPV];
        Row<DT>::decode(__builtin_nontemporal_load(xv + vi), t);
        fv(t);
    }
}

// f(x) for every element of the row
template <int DT, class F> __device__ __forceinline__ void row_for_each(const void* row, int64_t vocab, F f) {
    constexpr int EPV = Row<DT>::EPV;
    row_for_each_vec<DT>(
        row, vocab,
        [&](const float(&t)[EPV]) {
#pragma unroll
            for (int k = 0; k < EPV; ++k) f(t[k]);
        },
        f);
}

// out[i] = f(x[i], y[i], i) over one row; y may be NULL (then f receives 0 for it)
template <int DT, class F>
__device__ __forceinline__ void row_map(const void* xrow, const void* yrow, void* out, int64_t vocab, F f) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const bool vec = vec_ok<DT>(xrow, vocab) && vec_ok<DT>(out, vocab) && (!yrow || vec_ok<DT>(yrow, vocab));
    if (!vec) {
        for (int64_t i = tid; i < vocab; i += kDBlock)
            Row<DT>::store1(out, i, f(Row<DT>::load1(xrow, i), yrow ? Row<DT>::load1(yrow, i) : 0.f, i));
        return;
    }
    const u32x4* xv = static_cast<const u32x4*>(xrow);
    const u32x4* yv = static_cast<const u32x4*>(yrow);
    u32x4* ov = static_cast<u32x4*>(out);
    const int64_t nvec = vocab / EPV;
    for (int64_t vi = tid; vi < nvec; vi += kDBlock) {
        float a[EPV], b[EPV], d[EPV];
        Row<DT>::decode(__builtin_nontemporal_load(xv + vi), a);
        if (yrow) Row<DT>::decode(__builtin_nontemporal_load(yv + vi), b);
#pragma unroll
        for (int k = 0; k < EPV; ++k) d[k] = f(a[k], yrow ? b[k] : 0.f, vi * EPV + k);
        __builtin_nontemporal_store(Row<DT>::encode(d), ov + vi);
    }
}

template <int DT> __device__ __forceinline__ void row_fill_zero(void* out, int64_t vocab) {
    row_map<DT>(out, nullptr, out, vocab, [](float, float, int64_t) { return 0.f; });
}

// online (max, sum exp, sum exp * (x - max)): enough for the log-sum-exp and for sum_v p_v x_v
struct Ent {
    float m, s, t;
};
__device__ __forceinline__ void ent_push(Ent& a, float x) {
    if (x > a.m) {  // (a batch of 8 with one rescale and no branch measured 4 % slower here, unlike in the soft cross entropy)
        const float d = a.m - x, e = fast_exp2(d * kLog2e);
        a.t = e * (a.t + d * a.s);
        a.s = e * a.s;
        a.m = x;
    }
    const float d = x - a.m, p = fast_exp2(d * kLog2e);
    a.s += p;
    a.t += p > 0.f ? p * d : 0.f;  // a -inf logit has probability 0 and adds nothing
}
__device__ __forceinline__ Ent ent_merge(Ent a, Ent b) {
    const float m = fmaxf(a.m, b.m), da = a.m - m, db = b.m - m;
    const float ea = fast_exp2(da * kLog2e), eb = fast_exp2(db * kLog2e);
    Ent r;
    r.m = m;
    r.s = a.s * ea + b.s * eb;
    r.t = ea * (a.t + da * a.s) + eb * (b.t + db * b.s);
    return r;
}
__device__ __forceinline__ Ent ent_block(Ent a, Ent* smem) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        Ent o;
        o.m = __shfl_xor(a.m, off, kWave);
        o.s = __shfl_xor(a.s, off, kWave);
        o.t = __shfl_xor(a.t, off, kWave);
        a = ent_merge(a, o);
    }
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) smem[w] = a;
    __syncthreads();
    Ent tot = smem[0];
#pragma unroll
    for (int i = 1; i < kDWaves; ++i) tot = ent_merge(tot, smem[i]);
    return tot;
}

// ---------------------------------------------------------------------------------------------
// sum_v p_v log p_v
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kDBlock) void neg_entropy_fwd_kernel(RowsView x, float* __restrict__ h_out, float* __restrict__ lse_out) {
    __shared__ Ent smem[kDWaves];
    const int64_t r = blockIdx.x;
    const char* row = row_ptr<DT>(x, r);
    Ent acc{-1e30f, 0.f, 0.f};
    row_for_each<DT>(row, x.vocab, [&](float v) { ent_push(acc, v); });
    const Ent tot = ent_block(acc, smem);
    if (threadIdx.x == 0) {
        const float log_s = logf(tot.s);
        h_out[r] = tot.t / tot.s - log_s;  // sum p (x - m) - log s
        lse_out[r] = tot.m + log_s;
    }
}

// d / dz of sum_v p_v log p_v, times the upstream gradient: g * p_v * (log p_v - H)
template <int DT>
__global__ __launch_bounds__(kDBlock) void neg_entropy_bwd_kernel(RowsView x, const float* __restrict__ lse, const float* __restrict__ h,
                                                                  const float* __restrict__ grad, RowsView d) {
    const int64_t r = blockIdx.x;
    void* out = const_cast<char*>(row_ptr<DT>(d, r));
    const float g = grad[r];
    if (g == 0.f) { row_fill_zero<DT>(out, x.vocab); return; }
    const float l = lse[r], hh = h[r];
    row_map<DT>(row_ptr<DT>(x, r), nullptr, out, x.vocab, [&](float v, float, int64_t) {
        const float lp = v - l, p = fast_exp2(lp * kLog2e);
        return p > 0.f ? g * p * (lp - hh) : 0.f;
    });
}

// ---------------------------------------------------------------------------------------------
// log-probabilities at K given indices per row
// ---------------------------------------------------------------------------------------------
struct GatherArgs {
    const int64_t* idx;  // [rows, K]
    int64_t k, vstart, vend;
};

template <int DT>
__global__ __launch_bounds__(kDBlock) void gather_logprob_fwd_kernel(RowsView x, GatherArgs ga, float* __restrict__ out,
                                                                     float* __restrict__ lse_out) {
    __shared__ Lse smem[kDWaves];
    const int64_t r = blockIdx.x;
    const char* row = row_ptr<DT>(x, r);
    Lse acc{-FLT_MAX, 0.f};
    row_for_each_vec<DT>(
        row, x.vocab, [&](const float(&t)[Row<DT>::EPV]) { lse_push<Row<DT>::EPV>(acc, t); }, [&](float v) { lse_push1(acc, v); });
    const Lse tot = block_lse<kDWaves>(acc, smem);
    const float lse = tot.m + logf(tot.s);
    if (threadIdx.x == 0 && lse_out) lse_out[r] = lse;
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) {
        const int64_t gi = ga.idx[r * ga.k + j];
        out[r * ga.k + j] = (gi >= ga.vstart && gi < ga.vend) ? Row<DT>::load1(row, gi - ga.vstart) - lse : 0.f;
    }
}

// dz_v = -p_v * sum_k g_k + sum_{k: idx_k = v} g_k; the K touched elements are rewritten after the streaming
// pass with their complete value (every duplicate of an index computes and writes the same number)
template <int DT>
__global__ __launch_bounds__(kDBlock) void gather_logprob_bwd_kernel(RowsView x, GatherArgs ga, const float* __restrict__ lse,
                                                                     const float* __restrict__ grad, RowsView d) {
    __shared__ float sm[kDWaves];
    const int64_t r = blockIdx.x;
    const char* row = row_ptr<DT>(x, r);
    void* out = const_cast<char*>(row_ptr<DT>(d, r));
    float part = 0.f;
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) part += grad[r * ga.k + j];
    const float gsum = block_sum<float, kDWaves>(part, sm);
    const float l = lse[r];
    row_map<DT>(row, nullptr, out, x.vocab, [&](float v, float, int64_t) { return -fast_exp2((v - l) * kLog2e) * gsum; });
    __syncthreads();  // the streaming stores of this workgroup are visible to it before the patches land
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) {
        const int64_t gi = ga.idx[r * ga.k + j];
        if (gi < ga.vstart || gi >= ga.vend) continue;
        float add = 0.f;
        for (int64_t q = 0; q < ga.k; ++q) add += ga.idx[r * ga.k + q] == gi ? grad[r * ga.k + q] : 0.f;
        const float v = Row<DT>::load1(row, gi - ga.vstart);
        Row<DT>::store1(out, gi - ga.vstart, -fast_exp2((v - l) * kLog2e) * gsum + add);
    }
}

// ---------------------------------------------------------------------------------------------
// soft-target cross entropy  -sum_v softmax(y)_v * log_softmax(x)_v  = lse(x) - sum_v softmax(y)_v x_v
// ---------------------------------------------------------------------------------------------
struct Ce {
    float m, s, u;  // teacher max, sum exp(y - m), sum exp(y - m) * x
};
__device__ __forceinline__ void ce_push(Ce& a, float y, float x) {
    if (y > a.m) {
        const float e = fast_exp2((a.m - y) * kLog2e);
        a.s *= e;
        a.u *= e;
        a.m = y;
    }
    const float p = fast_exp2((y - a.m) * kLog2e);
    a.s += p;
    a.u += p > 0.f ? p * x : 0.f;
}
// N elements at once: one rescale for the batch's maximum instead of a branch and a rescale per new maximum
template <int N> __device__ __forceinline__ void ce_push_n(Ce& a, const float (&y)[N], const float (&x)[N]) {
    float vm = y[0];
#pragma unroll
    for (int k = 1; k < N; ++k) vm = fmaxf(vm, y[k]);
    const float mn = fmaxf(a.m, vm);
    const float e = fast_exp2((a.m - mn) * kLog2e);
    const float mn2 = mn * kLog2e;
    float s = a.s * e, u = a.u * e;
#pragma unroll
    for (int k = 0; k < N; ++k) {
        const float p = fast_exp2(__builtin_fmaf(y[k], kLog2e, -mn2));
        s += p;
        u += p > 0.f ? p * x[k] : 0.f;
    }
    a.m = mn;
    a.s = s;
    a.u = u;
}
__device__ __forceinline__ Ce ce_merge(Ce a, Ce b) {
    const float m = fmaxf(a.m, b.m);
    const float ea = fast_exp2((a.m - m) * kLog2e), eb = fast_exp2((b.m - m) * kLog2e);
    return Ce{m, a.s * ea + b.s * eb, a.u * ea + b.u * eb};
}

template <int DT>
__global__ __launch_bounds__(kDBlock) void soft_ce_fwd_kernel(RowsView x, RowsView y, float* __restrict__ ce_out,
                                                              float* __restrict__ lse_x_out, float* __restrict__ lse_y_out) {
    constexpr int EPV = Row<DT>::EPV;
    __shared__ Lse smem[kDWaves];
    __shared__ Ce smem_c[kDWaves];
    const int64_t r = blockIdx.x;
    const char* xr = row_ptr<DT>(x, r);
    const char* yr = row_ptr<DT>(y, r);
    const int tid = threadIdx.x;
    Lse ax{-FLT_MAX, 0.f};
    Ce ay{-1e30f, 0.f, 0.f};
    if (vec_ok<DT>(xr, x.vocab) && vec_ok<DT>(yr, x.vocab)) {
        const u32x4* xv = reinterpret_cast<const u32x4*>(xr);
        const u32x4* yv = reinterpret_cast<const u32x4*>(yr);
        const int64_t nvec = x.vocab / EPV;
        auto fold = [&](const u32x4& qx, const u32x4& qy) {
            float a[EPV], b[EPV];
            Row<DT>::decode(qx, a);
            Row<DT>::decode(qy, b);
            lse_push<EPV>(ax, a);
            ce_push_n<EPV>(ay, b, a);
        };
        int64_t base = 0;
        for (; base + kDUnroll * kDBlock <= nvec; base += kDUnroll * kDBlock) {
            u32x4 qx[kDUnroll], qy[kDUnroll];
#pragma unroll
            for (int u = 0; u < kDUnroll; ++u) {
                qx[u] = __builtin_nontemporal_load(xv + base + u * kDBlock + tid);
                qy[u] = __builtin_nontemporal_load(yv + base + u * kDBlock + tid);
            }
#pragma unroll
            for (int u = 0; u < kDUnroll; ++u) fold(qx[u], qy[u]);
        }
        for (int64_t vi = base + tid; vi < nvec; vi += kDBlock) fold(__builtin_nontemporal_load(xv + vi), __builtin_nontemporal_load(yv + vi));
    } else {
        for (int64_t i = tid; i < x.vocab; i += kDBlock) {
            const float a = Row<DT>::load1(xr, i), b = Row<DT>::load1(yr, i);
            lse_push1(ax, a);
            ce_push(ay, b, a);
        }
    }
    const Lse tx = block_lse<kDWaves>(ax, smem);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        Ce o{__shfl_xor(ay.m, off, kWave), __shfl_xor(ay.s, off, kWave), __shfl_xor(ay.u, off, kWave)};
        ay = ce_merge(ay, o);
    }
    if ((tid & (kWave - 1)) == 0) smem_c[tid / kWave] = ay;
    __syncthreads();
    if (tid == 0) {
        Ce ty = smem_c[0];
#pragma unroll
        for (int i = 1; i < kDWaves; ++i) ty = ce_merge(ty, smem_c[i]);
        const float lse_x = tx.m + logf(tx.s);
        ce_out[r] = lse_x - ty.u / ty.s;
        lse_x_out[r] = lse_x;
        lse_y_out[r] = ty.m + logf(ty.s);
    }
}

// d H(p, q) / d student logits = g * (q_v - p_v)
template <int DT>
__global__ __launch_bounds__(kDBlock) void soft_ce_bwd_kernel(RowsView x, RowsView y, const float* __restrict__ lse_x,
                                                              const float* __restrict__ lse_y, const float* __restrict__ grad, RowsView d) {
    const int64_t r = blockIdx.x;
    void* out = const_cast<char*>(row_ptr<DT>(d, r));
    const float g = grad[r];
    if (g == 0.f) { row_fill_zero<DT>(out, x.vocab); return; }
    const float lx = lse_x[r], ly = lse_y[r];
    row_map<DT>(row_ptr<DT>(x, r), row_ptr<DT>(y, r), out, x.vocab, [&](float a, float b, int64_t) {
        return g * (fast_exp2((a - lx) * kLog2e) - fast_exp2((b - ly) * kLog2e));
    });
}

// ---------------------------------------------------------------------------------------------
// log-softmax over K selected logits of a row: the K given vocabulary indices (the teacher's top-k) or,
// without indices, the row as it is (K = vocab).  The backward scatters into a zero-filled row.
// ---------------------------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(kDBlock) void topk_logsoftmax_fwd_kernel(RowsView x, GatherArgs ga, float* __restrict__ out) {
    __shared__ Lse smem[kDWaves];
    const int64_t r = blockIdx.x;
    const char* row = row_ptr<DT>(x, r);
    auto value = [&](int64_t j) -> float {
        if (!ga.idx) return Row<DT>::load1(row, j);
        const int64_t gi = ga.idx[r * ga.k + j];
        return (gi >= ga.vstart && gi < ga.vend) ? Row<DT>::load1(row, gi - ga.vstart) : -INFINITY;
    };
    Lse a{-FLT_MAX, 0.f};
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) lse_push1(a, value(j));
    const Lse t = block_lse<kDWaves>(a, smem);
    const float lse = t.m + logf(t.s);
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) out[r * ga.k + j] = value(j) - lse;
}

// d x[idx_j] = sum over duplicates of (g_j - exp(lp_j) * sum_q g_q); every other element of the row is zero
template <int DT>
__global__ __launch_bounds__(kDBlock) void topk_logsoftmax_bwd_kernel(RowsView d, GatherArgs ga, const float* __restrict__ lp,
                                                                      const float* __restrict__ grad) {
    __shared__ float sm[kDWaves];
    const int64_t r = blockIdx.x;
    void* out = const_cast<char*>(row_ptr<DT>(d, r));
    float part = 0.f;
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) part += grad[r * ga.k + j];
    const float gsum = block_sum<float, kDWaves>(part, sm);
    row_fill_zero<DT>(out, d.vocab);
    __syncthreads();  // the zero fill of this workgroup is visible to it before the K values land
    for (int64_t j = threadIdx.x; j < ga.k; j += kDBlock) {
        const int64_t gi = ga.idx[r * ga.k + j];
        if (gi < ga.vstart || gi >= ga.vend) continue;
        float add = 0.f;
        for (int64_t q = 0; q < ga.k; ++q)
            add += ga.idx[r * ga.k + q] == gi ? grad[r * ga.k + q] - expf(lp[r * ga.k + q]) * gsum : 0.f;
        Row<DT>::store1(out, gi - ga.vstart, add);
    }
}

// ---------------------------------------------------------------------------------------------
// distillation loss on top-k log-probabilities: forward / reverse / mixed KL per token over the K entries,
// plus the correction for the mass outside the top-k, masked mean over the tokens; loss and gradients in
// one pass.  One wave per token; a workgroup's four token sums go to one partial, the partials are added
// in index order by the finish kernel.
// ---------------------------------------------------------------------------------------------
struct KdArgs {
    const float* s_lp;         // [tokens, K] student log-probabilities
    const float* t_lp;         // [tokens, K] teacher log-probabilities
    const float* h_all;        // [tokens] sum_v p log p of the student's full row, or NULL
    const float* token_mask;   // [B, n] with row stride, or NULL (plain mean over the tokens)
    const float* sample_mask;  // [B]
    const float* global_valid; // [1] = valid tokens (index 1 of the usual pair)
    int64_t batch, n, k, tm_stride;
    int kl_type;               // 0 forward, 1 reverse, 2 mixed
    float w, log_infinitesimal;
    int correct;               // add the outside-top-k term
    float* d_s;                // [tokens, K]
    float* d_h;                // [tokens] or NULL
    double* parts;             // one per workgroup
    float* loss;
};

__global__ __launch_bounds__(kDBlock) void distill_topk_loss_kernel(KdArgs a) {
    __shared__ double sm[kDWaves];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t tokens = a.batch * a.n;
    const int64_t tok = static_cast<int64_t>(blockIdx.x) * kDWaves + wave;
    double contrib = 0.0;
    if (tok < tokens) {
        const int64_t b = tok / a.n, t = tok - b * a.n;
        const float den = a.token_mask ? a.global_valid[0] + 1e-8f : static_cast<float>(tokens);
        const float mask = a.token_mask ? a.token_mask[b * a.tm_stride + t] * a.sample_mask[b] : 1.f;
        const float wt = mask / den;  // d loss / d per-token value
        const float wf = a.kl_type == 0 ? 1.f : a.kl_type == 1 ? 0.f : a.w;  // weight of the forward term
        const float wr = 1.f - wf;                                            // ... of the reverse term
        const float c = a.correct ? (a.kl_type == 2 ? 1.f - a.w : 1.f) : 0.f;
        const float* sl = a.s_lp + tok * a.k;
        const float* tl = a.t_lp + tok * a.k;
        float fwd = 0.f, rev = 0.f, sp_slp = 0.f, sp_sum = 0.f;
        for (int64_t j = lane; j < a.k; j += kWave) {
            const float s = sl[j], u = tl[j];
            const float sp = expf(s), tp = expf(u);
            fwd += tp * (u - s);
            rev += sp * (s - u);
            sp_slp += sp * s;
            sp_sum += sp;
            float g = wf * -tp + wr * sp * (s - u + 1.f);
            if (a.correct) g -= c * sp * (s + 1.f - a.log_infinitesimal);
            a.d_s[tok * a.k + j] = wt * g;
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) {
            fwd += __shfl_xor(fwd, off, kWave);
            rev += __shfl_xor(rev, off, kWave);
            sp_slp += __shfl_xor(sp_slp, off, kWave);
            sp_sum += __shfl_xor(sp_sum, off, kWave);
        }
        float per_token = wf * fwd + wr * rev;
        if (a.correct) {
            const float h_rest = a.h_all[tok] - sp_slp, p_rest = 1.f - sp_sum;
            per_token += c * (h_rest - a.log_infinitesimal * p_rest);
        }
        if (lane == 0) {
            if (a.d_h) a.d_h[tok] = wt * c;
            contrib = static_cast<double>(per_token * mask);
        }
    }
    if (lane == 0) sm[wave] = contrib;
    __syncthreads();
    if (threadIdx.x == 0) {
        double tot = 0.0;
#pragma unroll
        for (int w = 0; w < kDWaves; ++w) tot += sm[w];
        a.parts[blockIdx.x] = tot;
    }
}

__global__ __launch_bounds__(kDBlock) void distill_topk_finish_kernel(KdArgs a, int64_t n_parts) {
    __shared__ double sm[kDWaves];
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < n_parts; i += kDBlock) acc += a.parts[i];
    acc = block_sum<double, kDWaves>(acc, sm);
    if (threadIdx.x == 0) {
        const float den = a.token_mask ? a.global_valid[0] + 1e-8f : static_cast<float>(a.batch * a.n);
        *a.loss = static_cast<float>(acc) / den;
    }
}

static int check_view(const nrl_rows* r) {
    if (!r) return fail(NRL_E_INVALID, "rows is NULL");
    if (r->dtype != NRL_F32 && r->dtype != NRL_BF16 && r->dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown logits dtype %d", r->dtype);
    if (r->n_outer < 0 || r->n_inner < 0 || r->vocab <= 0) return fail(NRL_E_INVALID, "bad shape");
    if (r->n_outer * r->n_inner > 0 && !r->logits) return fail(NRL_E_INVALID, "null logits");
    if (r->n_outer * r->n_inner >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    return NRL_OK;
}

static RowsView view_of(const nrl_rows* r) { return RowsView{r->logits, r->n_inner, r->vocab, r->stride_outer, r->stride_inner}; }
static RowsView view_of(const nrl_rows* r, const void* p, int64_t so, int64_t si) { return RowsView{p, r->n_inner, r->vocab, so, si}; }

}  // namespace nrl

using namespace nrl;

#define NRL_DT_DISPATCH(DTV, ...)                                   \
    switch (DTV) {                                                  \
        case NRL_F32: { constexpr int DT = NRL_F32; __VA_ARGS__; break; }  \
        case NRL_BF16: { constexpr int DT = NRL_BF16; __VA_ARGS__; break; } \
        default: { constexpr int DT = NRL_F16; __VA_ARGS__; break; }        \
    }

extern "C" int nrl_neg_entropy_fwd(const nrl_rows* rows, float* h_out, float* lse_out, void* stream) {
    if (int e = check_view(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (n == 0) return NRL_OK;
    if (!h_out || !lse_out) return fail(NRL_E_INVALID, "null output");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsView x = view_of(rows);
    NRL_DT_DISPATCH(rows->dtype, neg_entropy_fwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, h_out, lse_out));
    return check_launch("neg_entropy_fwd");
}

extern "C" int nrl_neg_entropy_bwd(const nrl_rows* rows, const float* lse, const float* h, const float* grad, void* dlogits,
                                   int64_t d_stride_outer, int64_t d_stride_inner, void* stream) {
    if (int e = check_view(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (n == 0) return NRL_OK;
    if (!lse || !h || !grad || !dlogits) return fail(NRL_E_INVALID, "null argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsView x = view_of(rows), d = view_of(rows, dlogits, d_stride_outer, d_stride_inner);
    NRL_DT_DISPATCH(rows->dtype, neg_entropy_bwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, lse, h, grad, d));
    return check_launch("neg_entropy_bwd");
}

extern "C" int nrl_gather_logprob_fwd(const nrl_rows* rows, const int64_t* indices, int64_t k, float* out, float* lse_out,
                                      void* stream) {
    if (int e = check_view(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (k < 0) return fail(NRL_E_INVALID, "negative K");
    if (n == 0 || k == 0) return NRL_OK;
    if (!indices || !out) return fail(NRL_E_INVALID, "null argument");
    if (rows->vocab_end - rows->vocab_start != rows->vocab) return fail(NRL_E_INVALID, "vocab range does not span the columns");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsView x = view_of(rows);
    const GatherArgs ga{indices, k, rows->vocab_start, rows->vocab_end};
    NRL_DT_DISPATCH(rows->dtype, gather_logprob_fwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, ga, out, lse_out));
    return check_launch("gather_logprob_fwd");
}

extern "C" int nrl_gather_logprob_bwd(const nrl_rows* rows, const int64_t* indices, int64_t k, const float* lse, const float* grad,
                                      void* dlogits, int64_t d_stride_outer, int64_t d_stride_inner, void* stream) {
    if (int e = check_view(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (k < 0) return fail(NRL_E_INVALID, "negative K");
    if (n == 0) return NRL_OK;
    if (!lse || !dlogits || (k > 0 && (!indices || !grad))) return fail(NRL_E_INVALID, "null argument");
    if (rows->vocab_end - rows->vocab_start != rows->vocab) return fail(NRL_E_INVALID, "vocab range does not span the columns");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsView x = view_of(rows), d = view_of(rows, dlogits, d_stride_outer, d_stride_inner);
    const GatherArgs ga{indices, k, rows->vocab_start, rows->vocab_end};
    NRL_DT_DISPATCH(rows->dtype, gather_logprob_bwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, ga, lse, grad, d));
    return check_launch("gather_logprob_bwd");
}

extern "C" int nrl_soft_cross_entropy_fwd(const nrl_rows* student, const void* teacher, int64_t t_stride_outer,
                                          int64_t t_stride_inner, float* ce_out, float* lse_student_out, float* lse_teacher_out,
                                          void* stream) {
    if (int e = check_view(student)) return e;
    const int64_t n = student->n_outer * student->n_inner;
    if (n == 0) return NRL_OK;
    if (!teacher || !ce_out || !lse_student_out || !lse_teacher_out) return fail(NRL_E_INVALID, "null argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsView x = view_of(student), y = view_of(student, teacher, t_stride_outer, t_stride_inner);
    NRL_DT_DISPATCH(student->dtype,
                    soft_ce_fwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, y, ce_out, lse_student_out, lse_teacher_out));
    return check_launch("soft_cross_entropy_fwd");
}

extern "C" int nrl_soft_cross_entropy_bwd(const nrl_rows* student, const void* teacher, int64_t t_stride_outer,
                                          int64_t t_stride_inner, const float* lse_student, const float* lse_teacher,
                                          const float* grad, void* dlogits, int64_t d_stride_outer, int64_t d_stride_inner,
                                          void* stream) {
    if (int e = check_view(student)) return e;
    const int64_t n = student->n_outer * student->n_inner;
    if (n == 0) return NRL_OK;
    if (!teacher || !lse_student || !lse_teacher || !grad || !dlogits) return fail(NRL_E_INVALID, "null argument");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsView x = view_of(student), y = view_of(student, teacher, t_stride_outer, t_stride_inner);
    const RowsView d = view_of(student, dlogits, d_stride_outer, d_stride_inner);
    NRL_DT_DISPATCH(student->dtype,
                    soft_ce_bwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, y, lse_student, lse_teacher, grad, d));
    return check_launch("soft_cross_entropy_bwd");
}

extern "C" int nrl_topk_logsoftmax_fwd(const nrl_rows* rows, const int64_t* indices, int64_t k, float* out, void* stream) {
    if (int e = check_view(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (k < 0) return fail(NRL_E_INVALID, "negative K");
    if (!indices && k != rows->vocab) return fail(NRL_E_INVALID, "without indices K must be the row length");
    if (n == 0 || k == 0) return NRL_OK;
    if (!out) return fail(NRL_E_INVALID, "null output");
    if (rows->vocab_end - rows->vocab_start != rows->vocab) return fail(NRL_E_INVALID, "vocab range does not span the columns");
    const RowsView x = view_of(rows);
    const GatherArgs ga{indices, k, rows->vocab_start, rows->vocab_end};
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DT_DISPATCH(rows->dtype, topk_logsoftmax_fwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(x, ga, out));
    return check_launch("topk_logsoftmax_fwd");
}

extern "C" int nrl_topk_logsoftmax_bwd(const nrl_rows* rows, const int64_t* indices, int64_t k, const float* logprobs,
                                       const float* grad, void* dlogits, int64_t d_stride_outer, int64_t d_stride_inner,
                                       void* stream) {
    if (int e = check_view(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (k < 0) return fail(NRL_E_INVALID, "negative K");
    if (n == 0) return NRL_OK;
    if (!dlogits || (k > 0 && (!indices || !logprobs || !grad))) return fail(NRL_E_INVALID, "null argument");
    if (rows->vocab_end - rows->vocab_start != rows->vocab) return fail(NRL_E_INVALID, "vocab range does not span the columns");
    const RowsView d = view_of(rows, dlogits, d_stride_outer, d_stride_inner);
    const GatherArgs ga{indices, k, rows->vocab_start, rows->vocab_end};
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DT_DISPATCH(rows->dtype, topk_logsoftmax_bwd_kernel<DT><<<dim3((unsigned)n), dim3(kDBlock), 0, s>>>(d, ga, logprobs, grad));
    return check_launch("topk_logsoftmax_bwd");
}

extern "C" int64_t nrl_distill_topk_loss_workspace_bytes(int64_t batch, int64_t n) {
    const int64_t tokens = batch * n;
    return ((tokens + kDWaves - 1) / kDWaves + 1) * static_cast<int64_t>(sizeof(double));
}

extern "C" int nrl_distill_topk_loss_fwd_bwd(const float* student_logprobs, const float* teacher_logprobs, const float* h_all,
                                             const float* token_mask, int64_t token_mask_stride, const float* sample_mask,
                                             const float* global_valid_toks, int64_t batch, int64_t n, int64_t k,
                                             int32_t kl_type, float mixed_kl_weight, int32_t zero_outside_topk,
                                             float log_infinitesimal, float* loss_out, float* d_student_out, float* d_h_all_out,
                                             void* workspace, int64_t workspace_bytes, void* stream) {
    if (batch < 0 || n < 0 || k < 0) return fail(NRL_E_INVALID, "bad shape [%lld, %lld, %lld]", (long long)batch, (long long)n, (long long)k);
    if (kl_type < 0 || kl_type > 2) return fail(NRL_E_INVALID, "kl_type must be 0 (forward), 1 (reverse) or 2 (mixed)");
    if (!loss_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (workspace_bytes < nrl_distill_topk_loss_workspace_bytes(batch, n)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 7) return fail(NRL_E_INVALID, "workspace must be 8-byte aligned");
    const int64_t tokens = batch * n;
    if (tokens >= (1ll << 31) * kDWaves) return fail(NRL_E_INVALID, "too many tokens");
    const bool correct = zero_outside_topk && kl_type != 0;
    if (tokens * k > 0 && (!student_logprobs || !teacher_logprobs || !d_student_out)) return fail(NRL_E_INVALID, "null logprobs or gradient output");
    if (tokens > 0 && correct && !h_all) return fail(NRL_E_INVALID, "H_all is NULL");
    if (tokens > 0 && token_mask && (!sample_mask || !global_valid_toks)) return fail(NRL_E_INVALID, "null sample_mask or global_valid_toks");
    KdArgs a;
    a.s_lp = student_logprobs; a.t_lp = teacher_logprobs; a.h_all = h_all; a.token_mask = token_mask; a.sample_mask = sample_mask;
    a.global_valid = global_valid_toks; a.batch = batch; a.n = n; a.k = k; a.tm_stride = token_mask_stride;
    a.kl_type = kl_type; a.w = mixed_kl_weight; a.log_infinitesimal = log_infinitesimal; a.correct = correct;
    a.d_s = d_student_out; a.d_h = correct ? d_h_all_out : nullptr; a.parts = static_cast<double*>(workspace); a.loss = loss_out;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t n_parts = (tokens + kDWaves - 1) / kDWaves;
    if (n_parts > 0) distill_topk_loss_kernel<<<dim3((unsigned)n_parts), dim3(kDBlock), 0, s>>>(a);
    distill_topk_finish_kernel<<<dim3(1), dim3(kDBlock), 0, s>>>(a, n_parts);
    return check_launch("distill_topk_loss_fwd_bwd");
}

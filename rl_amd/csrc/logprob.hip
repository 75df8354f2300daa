// K1 / K2: vocabulary logits -> token logprob (forward) and softmax-minus-onehot gradient
// (backward) for gfx950.
//
// One workgroup of 256 threads (4 wave64) owns one logits row.  The forward is a single
// streaming pass: every lane reads 16-byte vectors (coalesced, 1 KiB per wave per load), keeps a
// running (max, sum-of-exp) pair in registers, and the pairs are merged with a wave butterfly and
// a 4-entry LDS exchange.  The reduction order of a row depends only on the vocabulary size,
// never on how many rows are in the launch, so a row's result is bit-identical whatever batch it
// arrives in.  The backward re-reads the row once and writes the gradient once, narrowing from
// fp32 with a single round-to-nearest-even; probabilities are never stored.
//
// Algorithmic HBM traffic: forward V*sizeof(logit) per row, backward 2*V*sizeof(logit) per row.

#include <float.h>

#include "common.hpp"

namespace nrl {

constexpr int kBlock = 256;  // one workgroup of 4 wave64 per row
constexpr int kWaves = kBlock / kWave;
constexpr int kUnroll = 4;   // 16-byte loads in flight per lane

// rows that are read and written in the same pass stream through non-temporal loads and stores; rows
// that are only written (zero gradients) use plain stores, which a pure write stream sustains faster
template <typename P> __device__ __forceinline__ u32x4 k2_load(const P* p) { return __builtin_nontemporal_load(p); }
template <typename P> __device__ __forceinline__ void k2_store(u32x4 v, P* p) { __builtin_nontemporal_store(v, p); }

// number of leading elements before the first 16-byte boundary of a row
template <int DT> __device__ __forceinline__ int64_t row_head(const void* row, int64_t vocab) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(row);
    const int64_t h = static_cast<int64_t>(((16 - (a & 15)) & 15) / Row<DT>::BYTES);
    return h < vocab ? h : vocab;
}

// Online log-sum-exp of one row; every thread returns the row's (max, sum).
template <int DT, int TEMP>
__device__ __forceinline__ Lse row_online_lse(const void* row, int64_t vocab, float tparam, Lse* smem) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    Lse acc;
    acc.m = -FLT_MAX;
    acc.s = 0.f;

    const int64_t head = row_head<DT>(row, vocab);
    const int64_t nvec = (vocab - head) / EPV;
    const u32x4* xv = reinterpret_cast<const u32x4*>(static_cast<const char*>(row) + head * Row<DT>::BYTES);

    int64_t base = 0;
    for (; base + kUnroll * kBlock <= nvec; base += kUnroll * kBlock) {
        u32x4 r[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) r[u] = __builtin_nontemporal_load(xv + base + u * kBlock + tid);
        float v[kUnroll * EPV];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            float t[EPV];
            Row<DT>::decode(r[u], t);
#pragma unroll
            for (int k = 0; k < EPV; ++k) v[u * EPV + k] = scale_logit<DT, TEMP>(t[k], tparam);
        }
        lse_push<kUnroll * EPV>(acc, v);
    }
    for (int64_t i = base + tid; i < nvec; i += kBlock) {
        float t[EPV];
        Row<DT>::decode(__builtin_nontemporal_load(xv + i), t);
#pragma unroll
        for (int k = 0; k < EPV; ++k) t[k] = scale_logit<DT, TEMP>(t[k], tparam);
        lse_push<EPV>(acc, t);
    }
    // unaligned head and the tail shorter than one vector
    if (tid < head) lse_push1(acc, scale_logit<DT, TEMP>(Row<DT>::load1(row, tid), tparam));
    const int64_t tail0 = head + nvec * EPV;
    if (tail0 + tid < vocab) lse_push1(acc, scale_logit<DT, TEMP>(Row<DT>::load1(row, tail0 + tid), tparam));

    return block_lse<kWaves>(acc, smem);
}

template <int DT> __device__ __forceinline__ void row_zero(void* row, int64_t vocab) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const int64_t head = row_head<DT>(row, vocab);
    const int64_t nvec = (vocab - head) / EPV;
    u32x4* ov = reinterpret_cast<u32x4*>(static_cast<char*>(row) + head * Row<DT>::BYTES);
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int64_t i = tid; i < nvec; i += kBlock) ov[i] = z;
    if (tid < head) Row<DT>::store1(row, tid, 0.f);
    const int64_t tail0 = head + nvec * EPV;
    if (tail0 + tid < vocab) Row<DT>::store1(row, tail0 + tid, 0.f);
}

template <int DT, int TEMP>
__device__ __forceinline__ void row_write_grad(const void* row, void* out, int64_t vocab, float lse, float g,
                                               int64_t tgt, float tparam) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const RowGrad rg(lse, g, tparam);
    const int64_t head = row_head<DT>(row, vocab);
    if (row_head<DT>(out, vocab) != head) {
        // input and output rows are not congruent modulo 16 bytes: element-wise path
        for (int64_t i = tid; i < vocab; i += kBlock)
            Row<DT>::store1(out, i, grad_elem<DT, TEMP>(Row<DT>::load1(row, i), i == tgt, rg));
        return;
    }
    const int64_t nvec = (vocab - head) / EPV;
    const u32x4* xv = reinterpret_cast<const u32x4*>(static_cast<const char*>(row) + head * Row<DT>::BYTES);
    u32x4* ov = reinterpret_cast<u32x4*>(static_cast<char*>(out) + head * Row<DT>::BYTES);
    const int64_t tvec = tgt >= head ? (tgt - head) / EPV : -1;  // vector that holds the target
    const int tsub = tgt >= head ? static_cast<int>((tgt - head) % EPV) : -1;

    int64_t base = 0;
    for (; base + kUnroll * kBlock <= nvec; base += kUnroll * kBlock) {
        u32x4 r[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) r[u] = k2_load(xv + base + u * kBlock + tid);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int64_t vi = base + u * kBlock + tid;
            k2_store(grad_vec<DT, TEMP>(r[u], vi == tvec ? tsub : -1, rg), ov + vi);
        }
    }
    for (int64_t vi = base + tid; vi < nvec; vi += kBlock)
        k2_store(grad_vec<DT, TEMP>(k2_load(xv + vi), vi == tvec ? tsub : -1, rg), ov + vi);
    if (tid < head) Row<DT>::store1(out, tid, grad_elem<DT, TEMP>(Row<DT>::load1(row, tid), tid == tgt, rg));
    const int64_t tail0 = head + nvec * EPV;
    if (tail0 + tid < vocab) {
        const int64_t i = tail0 + tid;
        Row<DT>::store1(out, i, grad_elem<DT, TEMP>(Row<DT>::load1(row, i), i == tgt, rg));
    }
}

// ---------------------------------------------------------------------------------------------
// strided [n_outer, n_inner] rows
// ---------------------------------------------------------------------------------------------
struct RowArgs {
    const void* logits;
    int64_t n_inner, vocab, stride_outer, stride_inner;
    const int64_t* targets;
    int64_t ts_outer, ts_inner, vstart, vend;
    float tparam;
};

template <int DT, int TEMP>
__global__ __launch_bounds__(kBlock) void logprob_fwd_kernel(RowArgs a, float* __restrict__ logprob,
                                                             float* __restrict__ lse_out) {
    __shared__ Lse smem[kWaves];
    const int64_t r = blockIdx.x;
    const int64_t o = r / a.n_inner, i = r - o * a.n_inner;
    const char* row = static_cast<const char*>(a.logits) + (o * a.stride_outer + i * a.stride_inner) * Row<DT>::BYTES;
    const Lse t = row_online_lse<DT, TEMP>(row, a.vocab, a.tparam, smem);
    if (threadIdx.x == 0) {
        const float log_s = logf(t.s);
        const int64_t tg = a.targets[o * a.ts_outer + i * a.ts_inner];
        float lp = 0.f;
        if (tg >= a.vstart && tg < a.vend) {
            const float xt = scale_logit<DT, TEMP>(Row<DT>::load1(row, tg - a.vstart), a.tparam);
            lp = (xt - t.m) - log_s;
        }
        logprob[r] = lp;
        if (lse_out) lse_out[r] = t.m + log_s;
    }
}

// Forward-only logprobs in the [n_outer, n_inner + 1] shape handed to the driver: column 0 is zero, column i
// is the logprob of row i - 1, and everything at or past the sequence's length is zero; rows that only
// produce zeros are never read.
template <int DT, int TEMP>
__global__ __launch_bounds__(kBlock) void logprob_post_fwd_kernel(RowArgs a, const int64_t* __restrict__ lengths,
                                                                  float* __restrict__ out) {
    __shared__ Lse smem[kWaves];
    const int64_t r = blockIdx.x, cols = a.n_inner + 1;
    const int64_t o = r / cols, c = r - o * cols;
    if (c == 0 || c >= lengths[o]) {
        if (threadIdx.x == 0) out[r] = 0.f;
        return;
    }
    const int64_t i = c - 1;
    const char* row = static_cast<const char*>(a.logits) + (o * a.stride_outer + i * a.stride_inner) * Row<DT>::BYTES;
    const Lse t = row_online_lse<DT, TEMP>(row, a.vocab, a.tparam, smem);
    if (threadIdx.x == 0) {
        const int64_t tg = a.targets[o * a.ts_outer + i * a.ts_inner];
        float lp = 0.f;
        if (tg >= a.vstart && tg < a.vend) {
            const float xt = scale_logit<DT, TEMP>(Row<DT>::load1(row, tg - a.vstart), a.tparam);
            lp = (xt - t.m) - logf(t.s);
        }
        out[r] = lp;
    }
}

struct GradArgs {
    const float* lse;
    const float* grad;
    int64_t gs_outer, gs_inner;
    void* dlogits;
    int64_t d_n_inner, ds_outer, ds_inner;
};

template <int DT, int TEMP>
__global__ __launch_bounds__(kBlock) void logprob_bwd_kernel(RowArgs a, GradArgs ga) {
    const int64_t r = blockIdx.x;
    const int64_t o = r / ga.d_n_inner, i = r - o * ga.d_n_inner;
    char* out = static_cast<char*>(ga.dlogits) + (o * ga.ds_outer + i * ga.ds_inner) * Row<DT>::BYTES;
    float g = 0.f;
    if (i < a.n_inner) g = ga.grad[o * ga.gs_outer + i * ga.gs_inner];
    if (g == 0.f) {  // dropped position or masked token: the gradient row is exactly zero
        row_zero<DT>(out, a.vocab);
        return;
    }
    const char* row = static_cast<const char*>(a.logits) + (o * a.stride_outer + i * a.stride_inner) * Row<DT>::BYTES;
    const int64_t tg = a.targets[o * a.ts_outer + i * a.ts_inner];
    const int64_t tloc = (tg >= a.vstart && tg < a.vend) ? tg - a.vstart : -1;
    row_write_grad<DT, TEMP>(row, out, a.vocab, ga.lse[o * a.n_inner + i], g, tloc, a.tparam);
}

// ---------------------------------------------------------------------------------------------
// packed sequences: row p of a [T, V] buffer belongs to the sequence s with cu[s] <= p < cu[s+1]
// ---------------------------------------------------------------------------------------------
struct PackedArgs {
    const void* logits;
    int64_t total, vocab, row_stride;
    const int64_t* targets;
    int pre_rolled;
    const int32_t* cu;
    int64_t n_seq, unpacked_seqlen, vstart, vend;
    float tparam;
};


struct PackedPos {
    int64_t seq, pos, len, start;
};

__device__ __forceinline__ PackedPos locate(const PackedArgs& a, int64_t p, PackedPos* sh) {
    if (threadIdx.x == 0) {
        PackedPos q;
        q.seq = find_seq(a.cu, a.n_seq, p);
        q.start = q.seq >= 0 ? a.cu[q.seq] : 0;
        q.len = q.seq >= 0 ? a.cu[q.seq + 1] - q.start : 0;
        q.pos = p - q.start;
        *sh = q;
    }
    __syncthreads();
    return *sh;
}

__device__ __forceinline__ int64_t packed_target(const PackedArgs& a, const PackedPos& q) {
    const int64_t j = a.pre_rolled ? q.pos : (q.pos + 1 == q.len ? 0 : q.pos + 1);
    // (the targets hold at least `total` entries; boundaries that run past the packed row cannot index beyond them)
    const int64_t t = q.start + j;
    return a.targets[t < a.total ? t : a.total - 1];
}

template <int DT, int TEMP>
__global__ __launch_bounds__(kBlock) void logprob_packed_fwd_kernel(PackedArgs a, float* __restrict__ out,
                                                                    float* __restrict__ lse_out) {
    __shared__ Lse smem[kWaves];
    __shared__ PackedPos sh;
    const int64_t p = blockIdx.x;
    const PackedPos q = locate(a, p, &sh);
    // positions whose logprob is never used still get an LSE only when the caller keeps it
    const bool emitted = q.seq >= 0 && q.pos + 1 < q.len && q.pos < a.unpacked_seqlen - 1;
    if (!emitted) {
        if (lse_out && threadIdx.x == 0) lse_out[p] = 0.f;
        return;
    }
    const char* row = static_cast<const char*>(a.logits) + p * a.row_stride * Row<DT>::BYTES;
    const Lse t = row_online_lse<DT, TEMP>(row, a.vocab, a.tparam, smem);
    if (threadIdx.x == 0) {
        const float log_s = logf(t.s);
        const int64_t tg = packed_target(a, q);
        float lp = 0.f;
        if (tg >= a.vstart && tg < a.vend) {
            const float xt = scale_logit<DT, TEMP>(Row<DT>::load1(row, tg - a.vstart), a.tparam);
            lp = (xt - t.m) - log_s;
        }
        out[q.seq * (a.unpacked_seqlen - 1) + q.pos] = lp;
        if (lse_out) lse_out[p] = t.m + log_s;
    }
}

template <int DT, int TEMP>
__global__ __launch_bounds__(kBlock) void logprob_packed_bwd_kernel(PackedArgs a, const float* __restrict__ lse,
                                                                    const float* __restrict__ grad, void* dlogits,
                                                                    int64_t d_row_stride) {
    __shared__ PackedPos sh;
    const int64_t p = blockIdx.x;
    const PackedPos q = locate(a, p, &sh);
    char* out = static_cast<char*>(dlogits) + p * d_row_stride * Row<DT>::BYTES;
    const bool emitted = q.seq >= 0 && q.pos + 1 < q.len && q.pos < a.unpacked_seqlen - 1;
    const float g = emitted ? grad[q.seq * (a.unpacked_seqlen - 1) + q.pos] : 0.f;
    if (g == 0.f) {
        row_zero<DT>(out, a.vocab);
        return;
    }
    const char* row = static_cast<const char*>(a.logits) + p * a.row_stride * Row<DT>::BYTES;
    const int64_t tg = packed_target(a, q);
    const int64_t tloc = (tg >= a.vstart && tg < a.vend) ? tg - a.vstart : -1;
    row_write_grad<DT, TEMP>(row, out, a.vocab, lse[p], g, tloc, a.tparam);
}

// zero-fill of the unpacked [n_seq, L] output before the packed forward scatters into it
__global__ void fill_zero_f32(float* p, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
static int temp_code(float temperature, int mode, float* tparam) {
    if (temperature == 1.0f) { *tparam = 1.f; return 0; }
    if (mode == NRL_TEMP_DIV) { *tparam = temperature; return 1; }
    *tparam = 1.0f / temperature;
    return 2;
}

static int check_rows(const nrl_rows* r) {
    if (!r) return fail(NRL_E_INVALID, "rows is NULL");
    if (r->dtype != NRL_F32 && r->dtype != NRL_BF16 && r->dtype != NRL_F16)
        return fail(NRL_E_INVALID, "unknown logits dtype %d", r->dtype);
    if (r->n_outer < 0 || r->n_inner < 0 || r->vocab <= 0)
        return fail(NRL_E_INVALID, "bad shape [%lld, %lld, %lld]", (long long)r->n_outer, (long long)r->n_inner,
                    (long long)r->vocab);
    if (r->n_outer * r->n_inner > 0 && (!r->logits || !r->targets)) return fail(NRL_E_INVALID, "null logits or targets");
    if (r->vocab_end - r->vocab_start != r->vocab)
        return fail(NRL_E_INVALID, "vocab range [%lld, %lld) does not span %lld columns", (long long)r->vocab_start,
                    (long long)r->vocab_end, (long long)r->vocab);
    if (!(r->temperature > 0.f)) return fail(NRL_E_INVALID, "temperature must be positive");
    if (r->temp_mode != NRL_TEMP_DIV && r->temp_mode != NRL_TEMP_RCP) return fail(NRL_E_INVALID, "bad temp_mode");
    if (r->n_outer * r->n_inner >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    return NRL_OK;
}

static RowArgs make_row_args(const nrl_rows* r, float tparam) {
    RowArgs a;
    a.logits = r->logits;
    a.n_inner = r->n_inner;
    a.vocab = r->vocab;
    a.stride_outer = r->stride_outer;
    a.stride_inner = r->stride_inner;
    a.targets = r->targets;
    a.ts_outer = r->tgt_stride_outer;
    a.ts_inner = r->tgt_stride_inner;
    a.vstart = r->vocab_start;
    a.vend = r->vocab_end;
    a.tparam = tparam;
    return a;
}

// ---------------------------------------------------------------------------------------------
// log-softmax of whole rows, materialised (the stand-alone form of the stable log-softmax every logprob
// path starts from) and its backward dx_v = g_v - exp(y_v) * sum_u g_u
// ---------------------------------------------------------------------------------------------
// out_v = f(in_v [, in2_v]) over one row, by 16-byte vectors when the rows are congruent modulo 16 bytes
template <int DT, bool TWO, typename F>
__device__ __forceinline__ void row_apply(const void* in, const void* in2, void* out, int64_t vocab, F f) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const int64_t head = row_head<DT>(in, vocab);
    if (row_head<DT>(out, vocab) != head || (TWO && row_head<DT>(in2, vocab) != head)) {
        for (int64_t i = tid; i < vocab; i += kBlock)
            Row<DT>::store1(out, i, f(Row<DT>::load1(in, i), TWO ? Row<DT>::load1(in2, i) : 0.f));
        return;
    }
    const int64_t nvec = (vocab - head) / EPV;
    const u32x4* av = reinterpret_cast<const u32x4*>(static_cast<const char*>(in) + head * Row<DT>::BYTES);
    const u32x4* bv = TWO ? reinterpret_cast<const u32x4*>(static_cast<const char*>(in2) + head * Row<DT>::BYTES) : nullptr;
    u32x4* ov = reinterpret_cast<u32x4*>(static_cast<char*>(out) + head * Row<DT>::BYTES);
    for (int64_t i = tid; i < nvec; i += kBlock) {
        float x[EPV], y[EPV], o[EPV];
        Row<DT>::decode(av[i], x);
        if (TWO) Row<DT>::decode(bv[i], y);
#pragma unroll
        for (int k = 0; k < EPV; ++k) o[k] = f(x[k], TWO ? y[k] : 0.f);
        ov[i] = Row<DT>::encode(o);
    }
    if (tid < head) Row<DT>::store1(out, tid, f(Row<DT>::load1(in, tid), TWO ? Row<DT>::load1(in2, tid) : 0.f));
    const int64_t tail0 = head + nvec * EPV;
    if (tail0 + tid < vocab)
        Row<DT>::store1(out, tail0 + tid, f(Row<DT>::load1(in, tail0 + tid), TWO ? Row<DT>::load1(in2, tail0 + tid) : 0.f));
}

// sum of one row's elements (fp32 partials per lane, fixed-order workgroup reduction), 16-byte vectors
template <int DT> __device__ __forceinline__ float row_sum(const void* row, int64_t vocab, float* smem) {
    constexpr int EPV = Row<DT>::EPV;
    const int tid = threadIdx.x;
    const int64_t head = row_head<DT>(row, vocab);
    const int64_t nvec = (vocab - head) / EPV;
    const u32x4* xv = reinterpret_cast<const u32x4*>(static_cast<const char*>(row) + head * Row<DT>::BYTES);
    float part = 0.f;
    for (int64_t i = tid; i < nvec; i += kBlock) {
        float t[EPV];
        Row<DT>::decode(xv[i], t);
#pragma unroll
        for (int k = 0; k < EPV; ++k) part += t[k];
    }
    if (tid < head) part += Row<DT>::load1(row, tid);
    const int64_t tail0 = head + nvec * EPV;
    if (tail0 + tid < vocab) part += Row<DT>::load1(row, tail0 + tid);
    return block_sum<float, kWaves>(part, smem);
}

template <int DT>
__global__ __launch_bounds__(kBlock) void log_softmax_fwd_kernel(const void* __restrict__ logits, int64_t vocab, int64_t row_stride,
                                                                 void* __restrict__ out, int64_t out_stride) {
    __shared__ Lse smem[kWaves];
    const int64_t r = blockIdx.x;
    const char* row = static_cast<const char*>(logits) + r * row_stride * Row<DT>::BYTES;
    char* o = static_cast<char*>(out) + r * out_stride * Row<DT>::BYTES;
    const Lse t = row_online_lse<DT, 0>(row, vocab, 1.0f, smem);
    const float m = t.m, log_s = logf(t.s);
    row_apply<DT, false>(row, nullptr, o, vocab, [&](float x, float) { return (x - m) - log_s; });
}

template <int DT>
__global__ __launch_bounds__(kBlock) void log_softmax_bwd_kernel(const void* __restrict__ logprobs, int64_t vocab, int64_t lp_stride,
                                                                 const void* __restrict__ grad, int64_t g_stride,
                                                                 void* __restrict__ dx, int64_t dx_stride) {
    __shared__ float smem[kWaves];
    const int64_t r = blockIdx.x;
    const char* y = static_cast<const char*>(logprobs) + r * lp_stride * Row<DT>::BYTES;
    const char* g = static_cast<const char*>(grad) + r * g_stride * Row<DT>::BYTES;
    char* d = static_cast<char*>(dx) + r * dx_stride * Row<DT>::BYTES;
    const float sum_g = row_sum<DT>(g, vocab, smem);
    row_apply<DT, true>(g, y, d, vocab, [&](float gv, float yv) { return gv - fast_exp2(yv * kLog2e) * sum_g; });
}

// dst = src * (factor[0] / divisor) over strided rows (dst may be src): fp32 product, one narrowing to the
// rows' dtype.  The factor lives on the device so that the host never waits for it; when dst is src and the
// quotient is exactly 1 every workgroup leaves after reading it and no row is touched.
template <int DT>
__global__ __launch_bounds__(kBlock) void scale_rows_kernel(const void* src, void* dst, int64_t n_rows, int64_t n_inner, int64_t vocab,
                                                            int64_t src_outer, int64_t src_inner, int64_t dst_outer,
                                                            int64_t dst_inner, const float* __restrict__ factor, float divisor) {
    const float f = factor[0] / divisor;
    if (f == 1.f && src == dst) return;
    // (a bounded grid walking the rows: the launch that finds nothing to do costs a few microseconds, not one
    // workgroup per row)
    for (int64_t r = blockIdx.x; r < n_rows; r += gridDim.x) {
        const int64_t o = r / n_inner, i = r - o * n_inner;
        const char* in = static_cast<const char*>(src) + (o * src_outer + i * src_inner) * Row<DT>::BYTES;
        char* out = static_cast<char*>(dst) + (o * dst_outer + i * dst_inner) * Row<DT>::BYTES;
        row_apply<DT, false>(in, nullptr, out, vocab, [&](float x, float) { return x * f; });
    }
}

#define NRL_DISPATCH(DT_, TC_, ...)                                                         \
    switch ((DT_) * 3 + (TC_)) {                                                            \
        case NRL_F32 * 3 + 0: { constexpr int DT = NRL_F32, TEMP = 0; __VA_ARGS__; break; }        \
        case NRL_F32 * 3 + 1: { constexpr int DT = NRL_F32, TEMP = 1; __VA_ARGS__; break; }        \
        case NRL_F32 * 3 + 2: { constexpr int DT = NRL_F32, TEMP = 2; __VA_ARGS__; break; }        \
        case NRL_BF16 * 3 + 0: { constexpr int DT = NRL_BF16, TEMP = 0; __VA_ARGS__; break; }      \
        case NRL_BF16 * 3 + 1: { constexpr int DT = NRL_BF16, TEMP = 1; __VA_ARGS__; break; }      \
        case NRL_BF16 * 3 + 2: { constexpr int DT = NRL_BF16, TEMP = 2; __VA_ARGS__; break; }      \
        case NRL_F16 * 3 + 0: { constexpr int DT = NRL_F16, TEMP = 0; __VA_ARGS__; break; }        \
        case NRL_F16 * 3 + 1: { constexpr int DT = NRL_F16, TEMP = 1; __VA_ARGS__; break; }        \
        default: { constexpr int DT = NRL_F16, TEMP = 2; __VA_ARGS__; break; }                     \
    }

}  // namespace nrl

using namespace nrl;

extern "C" int nrl_logprob_fwd(const nrl_rows* rows, float* logprob_out, float* lse_out, void* stream) {
    if (int e = check_rows(rows)) return e;
    const int64_t n = rows->n_outer * rows->n_inner;
    if (n == 0) return NRL_OK;
    if (!logprob_out) return fail(NRL_E_INVALID, "logprob_out is NULL");
    float tparam;
    const int tc = temp_code(rows->temperature, rows->temp_mode, &tparam);
    const RowArgs a = make_row_args(rows, tparam);
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DISPATCH(rows->dtype, tc, logprob_fwd_kernel<DT, TEMP><<<dim3((unsigned)n), dim3(kBlock), 0, s>>>(a, logprob_out, lse_out));
    return check_launch("logprob_fwd");
}

extern "C" int nrl_logprob_post_fwd(const nrl_rows* rows, const int64_t* lengths, float* out, void* stream) {
    if (int e = check_rows(rows)) return e;
    const int64_t n = rows->n_outer * (rows->n_inner + 1);
    if (rows->n_outer == 0) return NRL_OK;
    if (!lengths || !out) return fail(NRL_E_INVALID, "lengths or out is NULL");
    if (n >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 positions in one launch");
    float tparam;
    const int tc = temp_code(rows->temperature, rows->temp_mode, &tparam);
    const RowArgs a = make_row_args(rows, tparam);
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DISPATCH(rows->dtype, tc, logprob_post_fwd_kernel<DT, TEMP><<<dim3((unsigned)n), dim3(kBlock), 0, s>>>(a, lengths, out));
    return check_launch("logprob_post_fwd");
}

extern "C" int nrl_logprob_bwd(const nrl_rows* rows, const float* lse, const float* grad, int64_t grad_stride_outer,
                               int64_t grad_stride_inner, void* dlogits, int64_t d_n_inner, int64_t d_stride_outer,
                               int64_t d_stride_inner, void* stream) {
    if (int e = check_rows(rows)) return e;
    if (d_n_inner < rows->n_inner) return fail(NRL_E_INVALID, "d_n_inner %lld < n_inner %lld", (long long)d_n_inner,
                                               (long long)rows->n_inner);
    const int64_t n = rows->n_outer * d_n_inner;
    if (n == 0) return NRL_OK;
    if (n >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    if (!dlogits || (rows->n_outer * rows->n_inner > 0 && (!lse || !grad)))
        return fail(NRL_E_INVALID, "null lse, grad or dlogits");
    float tparam;
    const int tc = temp_code(rows->temperature, rows->temp_mode, &tparam);
    const RowArgs a = make_row_args(rows, tparam);
    GradArgs ga;
    ga.lse = lse;
    ga.grad = grad;
    ga.gs_outer = grad_stride_outer;
    ga.gs_inner = grad_stride_inner;
    ga.dlogits = dlogits;
    ga.d_n_inner = d_n_inner;
    ga.ds_outer = d_stride_outer;
    ga.ds_inner = d_stride_inner;
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DISPATCH(rows->dtype, tc, logprob_bwd_kernel<DT, TEMP><<<dim3((unsigned)n), dim3(kBlock), 0, s>>>(a, ga));
    return check_launch("logprob_bwd");
}

// ids [B, S] -> packed ids [total_out]: sequence s fills [cup[s], cup[s+1]) with its first min(cu[s+1] - cu[s], S)
// ids, rolled by `shift` inside that span (element j comes from (j - shift) mod span), zero elsewhere.
__global__ __launch_bounds__(256) void pack_ids_kernel(const int64_t* ids, int64_t batch, int64_t width, int64_t ids_stride,
                                                       const int32_t* cu, const int32_t* cup, int64_t shift, int64_t* out,
                                                       int64_t total_out) {
    const int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (p >= total_out) return;
    int64_t v = 0;
    const int64_t s = find_seq(cup, batch, p);
    if (s >= 0) {
        const int64_t start = cup[s], span = cup[s + 1] - start;  // span >= 1: p lies inside it
        int64_t n_real = static_cast<int64_t>(cu[s + 1]) - cu[s];
        n_real = n_real < width ? n_real : width;
        int64_t src = (p - start - shift) % span;
        if (src < 0) src += span;
        if (src < n_real) v = ids[s * ids_stride + src];
    }
    out[p] = v;
}

static int check_packed(const void* logits, int32_t dtype, int64_t total, int64_t vocab, const int64_t* targets,
                        const int32_t* cu, int64_t n_seq, int64_t unpacked_seqlen, int64_t vstart, int64_t vend,
                        float temperature, int32_t temp_mode) {
    if (dtype != NRL_F32 && dtype != NRL_BF16 && dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown logits dtype %d", dtype);
    if (total < 0 || vocab <= 0 || n_seq < 0 || unpacked_seqlen < 1) return fail(NRL_E_INVALID, "bad packed shape");
    if (total > 0 && (!logits || !targets || !cu)) return fail(NRL_E_INVALID, "null logits, targets or cu_seqlens");
    if (vend - vstart != vocab) return fail(NRL_E_INVALID, "vocab range does not span the columns");
    if (!(temperature > 0.f)) return fail(NRL_E_INVALID, "temperature must be positive");
    if (temp_mode != NRL_TEMP_DIV && temp_mode != NRL_TEMP_RCP) return fail(NRL_E_INVALID, "bad temp_mode");
    if (total >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    return NRL_OK;
}

extern "C" int nrl_logprob_packed_fwd(const void* logits, int32_t dtype, int64_t total_tokens, int64_t vocab,
                                      int64_t row_stride, const int64_t* targets, int32_t pre_rolled,
                                      const int32_t* cu_seqlens, int64_t n_seq, int64_t unpacked_seqlen,
                                      int64_t vocab_start, int64_t vocab_end, float temperature, int32_t temp_mode,
                                      float* out, float* lse_out, void* stream) {
    if (int e = check_packed(logits, dtype, total_tokens, vocab, targets, cu_seqlens, n_seq, unpacked_seqlen,
                             vocab_start, vocab_end, temperature, temp_mode))
        return e;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t n_out = n_seq * (unpacked_seqlen - 1);
    if (n_out > 0) {
        if (!out) return fail(NRL_E_INVALID, "out is NULL");
        fill_zero_f32<<<dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, s>>>(out, n_out);
    }
    if (total_tokens == 0 || n_out == 0) return check_launch("logprob_packed_fwd");
    PackedArgs a;
    a.logits = logits; a.total = total_tokens; a.vocab = vocab; a.row_stride = row_stride; a.targets = targets;
    a.pre_rolled = pre_rolled; a.cu = cu_seqlens; a.n_seq = n_seq; a.unpacked_seqlen = unpacked_seqlen;
    a.vstart = vocab_start; a.vend = vocab_end;
    const int tc = temp_code(temperature, temp_mode, &a.tparam);
    NRL_DISPATCH(dtype, tc,
                 logprob_packed_fwd_kernel<DT, TEMP><<<dim3((unsigned)total_tokens), dim3(kBlock), 0, s>>>(a, out, lse_out));
    return check_launch("logprob_packed_fwd");
}

extern "C" int nrl_logprob_packed_bwd(const void* logits, int32_t dtype, int64_t total_tokens, int64_t vocab,
                                      int64_t row_stride, const int64_t* targets, int32_t pre_rolled,
                                      const int32_t* cu_seqlens, int64_t n_seq, int64_t unpacked_seqlen,
                                      int64_t vocab_start, int64_t vocab_end, float temperature, int32_t temp_mode,
                                      const float* lse, const float* grad, void* dlogits, int64_t d_row_stride,
                                      void* stream) {
    if (int e = check_packed(logits, dtype, total_tokens, vocab, targets, cu_seqlens, n_seq, unpacked_seqlen,
                             vocab_start, vocab_end, temperature, temp_mode))
        return e;
    if (total_tokens == 0) return NRL_OK;
    if (!dlogits || !lse || (n_seq * (unpacked_seqlen - 1) > 0 && !grad)) return fail(NRL_E_INVALID, "null lse, grad or dlogits");
    PackedArgs a;
    a.logits = logits; a.total = total_tokens; a.vocab = vocab; a.row_stride = row_stride; a.targets = targets;
    a.pre_rolled = pre_rolled; a.cu = cu_seqlens; a.n_seq = n_seq; a.unpacked_seqlen = unpacked_seqlen;
    a.vstart = vocab_start; a.vend = vocab_end;
    const int tc = temp_code(temperature, temp_mode, &a.tparam);
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DISPATCH(dtype, tc,
                 logprob_packed_bwd_kernel<DT, TEMP><<<dim3((unsigned)total_tokens), dim3(kBlock), 0, s>>>(
                     a, lse, grad, dlogits, d_row_stride));
    return check_launch("logprob_packed_bwd");
}

extern "C" int nrl_log_softmax_fwd(const void* logits, int32_t dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                   void* out, int64_t out_row_stride, void* stream) {
    if (dtype != NRL_F32 && dtype != NRL_BF16 && dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown logits dtype %d", dtype);
    if (n_rows < 0 || vocab <= 0 || row_stride < vocab || out_row_stride < vocab) return fail(NRL_E_INVALID, "bad shape or stride");
    if (n_rows == 0) return NRL_OK;
    if (!logits || !out) return fail(NRL_E_INVALID, "null logits or out");
    if (n_rows >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DISPATCH(dtype, 0, (void)TEMP; log_softmax_fwd_kernel<DT><<<dim3((unsigned)n_rows), dim3(kBlock), 0, s>>>(logits, vocab, row_stride, out, out_row_stride));
    return check_launch("log_softmax_fwd");
}

extern "C" int nrl_log_softmax_bwd(const void* logprobs, int32_t dtype, int64_t n_rows, int64_t vocab, int64_t lp_row_stride,
                                   const void* grad, int64_t grad_row_stride, void* dx, int64_t dx_row_stride, void* stream) {
    if (dtype != NRL_F32 && dtype != NRL_BF16 && dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown dtype %d", dtype);
    if (n_rows < 0 || vocab <= 0 || lp_row_stride < vocab || grad_row_stride < vocab || dx_row_stride < vocab)
        return fail(NRL_E_INVALID, "bad shape or stride");
    if (n_rows == 0) return NRL_OK;
    if (!logprobs || !grad || !dx) return fail(NRL_E_INVALID, "null logprobs, grad or dx");
    if (n_rows >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    hipStream_t s = static_cast<hipStream_t>(stream);
    NRL_DISPATCH(dtype, 0, (void)TEMP; log_softmax_bwd_kernel<DT><<<dim3((unsigned)n_rows), dim3(kBlock), 0, s>>>(logprobs, vocab, lp_row_stride, grad,
                                                                                                   grad_row_stride, dx, dx_row_stride));
    return check_launch("log_softmax_bwd");
}

extern "C" int nrl_scale_rows(const void* src, void* dst, int32_t dtype, int64_t n_outer, int64_t n_inner, int64_t vocab,
                              int64_t src_stride_outer, int64_t src_stride_inner, int64_t dst_stride_outer,
                              int64_t dst_stride_inner, const float* factor, float divisor, void* stream) {
    if (dtype != NRL_F32 && dtype != NRL_BF16 && dtype != NRL_F16) return fail(NRL_E_INVALID, "unknown dtype %d", dtype);
    if (n_outer < 0 || n_inner < 0 || vocab <= 0) return fail(NRL_E_INVALID, "bad shape");
    if (!(divisor != 0.f)) return fail(NRL_E_INVALID, "divisor must not be zero");
    const int64_t n = n_outer * n_inner;
    if (n == 0) return NRL_OK;
    if (!src || !dst || !factor) return fail(NRL_E_INVALID, "null src, dst or factor");
    if (n >= (1ll << 31)) return fail(NRL_E_INVALID, "more than 2^31 rows in one launch");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int64_t kScaleGrid = 4096;  // 16 workgroups per compute unit; each walks its share of the rows
    NRL_DISPATCH(dtype, 0, (void)TEMP; scale_rows_kernel<DT><<<dim3((unsigned)(n < kScaleGrid ? n : kScaleGrid)), dim3(kBlock), 0, s>>>(
                                 src, dst, n, n_inner, vocab, src_stride_outer, src_stride_inner, dst_stride_outer,
                                 dst_stride_inner, factor, divisor));
    return check_launch("scale_rows");
}

extern "C" int nrl_pack_input_ids(const int64_t* input_ids, int64_t batch, int64_t width, int64_t row_stride,
                                  const int32_t* cu_seqlens, const int32_t* cu_seqlens_padded, int64_t roll_shift,
                                  int64_t* packed_out, int64_t total_out, void* stream) {
    if (batch < 0 || width < 0 || total_out < 0 || row_stride < width) return fail(NRL_E_INVALID, "pack_input_ids: bad shape");
    if (total_out == 0) return NRL_OK;
    if (!packed_out || !cu_seqlens || !cu_seqlens_padded || (batch * width > 0 && !input_ids))
        return fail(NRL_E_INVALID, "pack_input_ids: null pointer");
    pack_ids_kernel<<<dim3((unsigned)((total_out + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(
        input_ids, batch, width, row_stride, cu_seqlens, cu_seqlens_padded, roll_shift, packed_out, total_out);
    return check_launch("pack_input_ids");
}

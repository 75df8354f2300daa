// K6: fused lm_head -> token logprob (hidden @ W^T, never materialising the full logits) and its
// backward (dH, dW), on the gfx950 matrix cores.
//
// One bf16 MFMA GEMM core, C[M,N] = A[M,K] * B[N,K]^T with fp32 accumulation, serves every product:
//   * 256 x 128 output tile per workgroup (4 wave64 in a 2 x 2 grid, 128 x 64 per wave = 4 x 2
//     v_mfma_f32_32x32x16_bf16 tiles, 128 accumulator registers per lane);
//   * K is walked in 64-wide slabs: 16-byte global loads into registers for slab k+1 while slab k is
//     consumed from LDS (rows padded to 72 elements so the 16-byte fragment reads of 32 different
//     rows do not land on the same banks).
// Epilogues:
//   LSE    forward: the tile's logits are rounded to bf16 (the reference's matmul returns bf16) and
//          folded into a running (max, sum-exp) per row kept in registers while the workgroup walks
//          its vocabulary tiles; the target's logit is captured on the way.  Only [rows] sized partials
//          leave the chip.
//   GRAD   backward: recomputed tile -> g * (onehot - exp(x - lse)) written as bf16 both row-major
//          (for dH = G W) and transposed (for dW = G^T hidden) for one token chunk at a time.
//   STORE / ACCUM  plain fp32 C = or C += for dH and dW.
// The vocabulary is walked in tiles while the token chunk bounds what is materialised:
// chunk x V bf16 for G and G^T (1.2 GB each at chunk 4096, V 151936) instead of N x V.

#include <float.h>
#include <math.h>

#include "common.hpp"

namespace nrl {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GB_M = 256, GB_N = 128, GB_K = 64, GB_LD = GB_K + 8;  // LDS row stride (elements)
constexpr int GB_THREADS = 256;
constexpr int GB_A_LOADS = GB_M * GB_K / 8 / GB_THREADS;  // 8
constexpr int GB_B_LOADS = GB_N * GB_K / 8 / GB_THREADS;  // 4

struct GemmOperands {
    const uint16_t* a;  // [M, K] row stride lda
    const uint16_t* b;  // [N, K] row stride ldb
    int64_t lda, ldb, m, n, k;  // k multiple of 8; slabs beyond k read as zero
};

// accumulator element e (0..15) of lane l in a 32x32 tile: column l % 32, row 8*(e/4) + 4*(l/32) + e%4
__device__ __forceinline__ int acc_row(int e, int lane) { return 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3); }

struct GemmRegs {
    u32x4 a[GB_A_LOADS];
    u32x4 b[GB_B_LOADS];
};

__device__ __forceinline__ void gemm_load_slab(const GemmOperands& op, int64_t row0, int64_t col0, int64_t k0, GemmRegs& r) {
    const int tid = threadIdx.x;
    const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < GB_A_LOADS; ++j) {
        const int c = tid + GB_THREADS * j;
        const int rr = c >> 3, kc = c & 7;
        int64_t grow = row0 + rr;
        grow = grow < op.m ? grow : op.m - 1;
        const int64_t kk = k0 + kc * 8;
        r.a[j] = kk < op.k ? *reinterpret_cast<const u32x4*>(op.a + grow * op.lda + kk) : zero;
    }
#pragma unroll
    for (int j = 0; j < GB_B_LOADS; ++j) {
        const int c = tid + GB_THREADS * j;
        const int rr = c >> 3, kc = c & 7;
        int64_t grow = col0 + rr;
        grow = grow < op.n ? grow : op.n - 1;
        const int64_t kk = k0 + kc * 8;
        r.b[j] = kk < op.k ? *reinterpret_cast<const u32x4*>(op.b + grow * op.ldb + kk) : zero;
    }
}

__device__ __forceinline__ void gemm_store_slab(const GemmRegs& r, uint16_t* As, uint16_t* Bs) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int j = 0; j < GB_A_LOADS; ++j) {
        const int c = tid + GB_THREADS * j;
        *reinterpret_cast<u32x4*>(As + (c >> 3) * GB_LD + (c & 7) * 8) = r.a[j];
    }
#pragma unroll
    for (int j = 0; j < GB_B_LOADS; ++j) {
        const int c = tid + GB_THREADS * j;
        *reinterpret_cast<u32x4*>(Bs + (c >> 3) * GB_LD + (c & 7) * 8) = r.b[j];
    }
}

// acc[i][j] += A[row0.., :] * B[col0.., :]^T for the workgroup's 256 x 128 tile
__device__ __forceinline__ void gemm_tile(const GemmOperands& op, int64_t row0, int64_t col0, f32x16 (&acc)[4][2],
                                          uint16_t* As, uint16_t* Bs) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
    GemmRegs regs;
    const int64_t nk = (op.k + GB_K - 1) / GB_K;
    gemm_load_slab(op, row0, col0, 0, regs);
    __syncthreads();  // previous users of the LDS tiles are done
    gemm_store_slab(regs, As, Bs);
    __syncthreads();
    for (int64_t kt = 0; kt < nk; ++kt) {
        if (kt + 1 < nk) gemm_load_slab(op, row0, col0, (kt + 1) * GB_K, regs);
#pragma unroll
        for (int ks = 0; ks < GB_K / 16; ++ks) {
            bf16x8 af[4], bfr[2];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                af[i] = *reinterpret_cast<const bf16x8*>(As + (wm * 128 + i * 32 + frag_row) * GB_LD + ks * 16 + frag_k);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                bfr[j] = *reinterpret_cast<const bf16x8*>(Bs + (wn * 64 + j * 32 + frag_row) * GB_LD + ks * 16 + frag_k);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
        if (kt + 1 < nk) {
            gemm_store_slab(regs, As, Bs);
            __syncthreads();
        }
    }
}

__device__ __forceinline__ void zero_acc(f32x16 (&acc)[4][2]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
}

__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// ---------------------------------------------------------------------------------------------
// forward: running log-sum-exp over the vocabulary tiles of one split
// ---------------------------------------------------------------------------------------------
struct LmFwdArgs {
    GemmOperands op;           // a = hidden [N,H], b = W [V,H]
    const int64_t* targets;    // [N]
    int64_t vocab_start;       // target ids are global; columns are local
    int n_splits;
    float* part_m;             // [n_splits, N]
    float* part_s;             // [n_splits, N]
    float* xt;                 // [N] target logit (written by the tile that holds it)
};

__global__ __launch_bounds__(GB_THREADS) void lmhead_fwd_kernel(LmFwdArgs a) {
    __shared__ __attribute__((aligned(16))) uint16_t As[GB_M * GB_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[GB_N * GB_LD];
    __shared__ int tgt_local[GB_M];
    __shared__ float comb_m[2][GB_M], comb_s[2][GB_M];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * GB_M;
    const int split = blockIdx.y;
    const int64_t n_tiles = (a.op.n + GB_N - 1) / GB_N;
    {
        const int64_t grow = row0 + tid;
        int64_t t = -1;
        if (grow < a.op.m) t = a.targets[grow] - a.vocab_start;
        tgt_local[tid] = (t >= 0 && t < a.op.n) ? static_cast<int>(t) : -1;
    }
    float run_m[4][16], run_s[4][16];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) { run_m[i][e] = -FLT_MAX; run_s[i][e] = 0.f; }

    for (int64_t tile = split; tile < n_tiles; tile += a.n_splits) {
        const int64_t col0 = tile * GB_N;
        f32x16 acc[4][2];
        zero_acc(acc);
        gemm_tile(a.op, row0, col0, acc, As, Bs);
        const int64_t c0 = col0 + wn * 64 + (lane & 31), c1 = c0 + 32;
        const bool ok0 = c0 < a.op.n, ok1 = c1 < a.op.n;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int rl = wm * 128 + i * 32 + acc_row(e, lane);
                const float x0 = ok0 ? round_bf16(acc[i][0][e]) : -INFINITY;
                const float x1 = ok1 ? round_bf16(acc[i][1][e]) : -INFINITY;
                const float mn = fmaxf(run_m[i][e], fmaxf(x0, x1));
                run_s[i][e] = run_s[i][e] * fast_exp2((run_m[i][e] - mn) * kLog2e) + fast_exp2((x0 - mn) * kLog2e) +
                              fast_exp2((x1 - mn) * kLog2e);
                run_m[i][e] = mn;
                const int tg = tgt_local[rl];
                if (tg == c0) a.xt[row0 + rl] = x0;
                if (tg == c1) a.xt[row0 + rl] = x1;
            }
        }
    }
    // combine the 32 lanes that share a row, then the two column halves of the workgroup
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            float m = run_m[i][e], s = run_s[i][e];
#pragma unroll
            for (int off = 16; off > 0; off >>= 1) {
                const float om = __shfl_xor(m, off, kWave), os = __shfl_xor(s, off, kWave);
                const float mn = fmaxf(m, om);
                s = s * fast_exp2((m - mn) * kLog2e) + os * fast_exp2((om - mn) * kLog2e);
                m = mn;
            }
            if ((lane & 31) == 0) {
                const int rl = wm * 128 + i * 32 + acc_row(e, lane);
                comb_m[wn][rl] = m;
                comb_s[wn][rl] = s;
            }
        }
    }
    __syncthreads();
    {
        const int64_t grow = row0 + tid;
        if (grow < a.op.m) {
            const float m0 = comb_m[0][tid], m1 = comb_m[1][tid];
            const float mn = fmaxf(m0, m1);
            const float s = comb_s[0][tid] * fast_exp2((m0 - mn) * kLog2e) + comb_s[1][tid] * fast_exp2((m1 - mn) * kLog2e);
            a.part_m[static_cast<int64_t>(split) * a.op.m + grow] = mn;
            a.part_s[static_cast<int64_t>(split) * a.op.m + grow] = s;
        }
    }
}

__global__ void lmhead_fwd_finish_kernel(int64_t n, int n_splits, const float* part_m, const float* part_s, const float* xt,
                                         const int64_t* targets, int64_t vocab_start, int64_t vocab_end, float* logprob,
                                         float* lse_out) {
    const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (r >= n) return;
    float m = part_m[r], s = part_s[r];
    for (int k = 1; k < n_splits; ++k) {
        const float om = part_m[k * n + r], os = part_s[k * n + r];
        const float mn = fmaxf(m, om);
        s = s * fast_exp2((m - mn) * kLog2e) + os * fast_exp2((om - mn) * kLog2e);
        m = mn;
    }
    const float log_s = logf(s);
    const int64_t t = targets[r];
    logprob[r] = (t >= vocab_start && t < vocab_end) ? (xt[r] - m) - log_s : 0.f;
    if (lse_out) lse_out[r] = m + log_s;
}

// ---------------------------------------------------------------------------------------------
// backward: recompute a [chunk, V] slab of logits and emit G = g * (onehot - softmax) in both layouts
// ---------------------------------------------------------------------------------------------
struct LmGradArgs {
    GemmOperands op;         // a = hidden chunk [chunk, H], b = W [V, H]
    const int64_t* targets;  // [chunk]
    int64_t vocab_start;
    const float* lse;        // [chunk]
    const float* grad;       // [chunk] upstream d loss / d logprob
    uint16_t* g;             // [chunk_pad, ldg] row-major, columns >= V zero
    int64_t ldg;
    uint16_t* gt;            // [V, ldgt] transposed, columns >= chunk zero
    int64_t ldgt;
};

__global__ __launch_bounds__(GB_THREADS) void lmhead_grad_kernel(LmGradArgs a) {
    __shared__ __attribute__((aligned(16))) uint16_t As[GB_M * GB_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[GB_N * GB_LD];
    __shared__ int tgt_local[GB_M];
    __shared__ float lse_l[GB_M], g_l[GB_M];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * GB_M;
    const int64_t col0 = static_cast<int64_t>(blockIdx.y) * GB_N;
    {
        const int64_t grow = row0 + tid;
        int64_t t = -1;
        float l = 0.f, g = 0.f;
        if (grow < a.op.m) { t = a.targets[grow] - a.vocab_start; l = a.lse[grow]; g = a.grad[grow]; }
        tgt_local[tid] = (t >= 0 && t < a.op.n) ? static_cast<int>(t) : -1;
        lse_l[tid] = l;
        g_l[tid] = g;
    }
    f32x16 acc[4][2];
    zero_acc(acc);
    gemm_tile(a.op, row0, col0, acc, As, Bs);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int64_t c = col0 + wn * 64 + j * 32 + (lane & 31);
        const bool col_ok = c < a.op.n;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {  // four groups of four consecutive rows
                uint32_t packed[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int e = q * 4 + u;
                    const int rl = wm * 128 + i * 32 + acc_row(e, lane);
                    const bool row_ok = row0 + rl < a.op.m;
                    float gv = 0.f;
                    if (row_ok && col_ok) {
                        const float x = round_bf16(acc[i][j][e]);
                        const float p = fast_exp2((x - lse_l[rl]) * kLog2e);
                        gv = ((tgt_local[rl] == c ? 1.f : 0.f) - p) * g_l[rl];
                    }
                    packed[u] = f32_to_bf16_bits(gv);
                    if (c < a.ldg && row0 + rl < ((a.op.m + 63) / 64) * 64) a.g[(row0 + rl) * a.ldg + c] = static_cast<uint16_t>(packed[u]);
                }
                const int64_t r_first = row0 + wm * 128 + i * 32 + acc_row(q * 4, lane);
                if (col_ok && r_first < a.ldgt) {
                    uint2 v;
                    v.x = packed[0] | (packed[1] << 16);
                    v.y = packed[2] | (packed[3] << 16);
                    *reinterpret_cast<uint2*>(a.gt + c * a.ldgt + r_first) = v;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// plain GEMM with fp32 output: C = A B^T or C += A B^T
// ---------------------------------------------------------------------------------------------
template <bool ACCUM>
__global__ __launch_bounds__(GB_THREADS) void gemm_f32_kernel(GemmOperands op, float* c, int64_t ldc) {
    __shared__ __attribute__((aligned(16))) uint16_t As[GB_M * GB_LD];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[GB_N * GB_LD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * GB_M;
    const int64_t col0 = static_cast<int64_t>(blockIdx.y) * GB_N;
    f32x16 acc[4][2];
    zero_acc(acc);
    gemm_tile(op, row0, col0, acc, As, Bs);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t col = col0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t row = row0 + wm * 128 + i * 32 + acc_row(e, lane);
                if (row < op.m && col < op.n) {
                    float* p = c + row * ldc + col;
                    *p = ACCUM ? *p + acc[i][j][e] : acc[i][j][e];
                }
            }
        }
}

// dst[c, r] = src[r, c] for r < rows, c < cols; dst row stride ldd, columns [rows, pad_cols) zero-filled
__global__ void transpose_bf16_kernel(const uint16_t* src, int64_t rows, int64_t cols, int64_t lds_, uint16_t* dst,
                                      int64_t ldd, int64_t pad_cols) {
    __shared__ uint16_t tile[64][66];
    const int64_t r0 = static_cast<int64_t>(blockIdx.y) * 64, c0 = static_cast<int64_t>(blockIdx.x) * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 256 threads: 64 x 4
    for (int k = ty; k < 64; k += 4) {
        const int64_t r = r0 + k, c = c0 + tx;
        tile[k][tx] = (r < rows && c < cols) ? src[r * lds_ + c] : static_cast<uint16_t>(0);
    }
    __syncthreads();
    for (int k = ty; k < 64; k += 4) {
        const int64_t c = c0 + k, r = r0 + tx;
        if (c < cols && r < pad_cols) dst[c * ldd + r] = tile[tx][k];
    }
}

__global__ void f32_to_bf16_kernel(const float* src, uint16_t* dst, int64_t n) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        dst[i] = static_cast<uint16_t>(f32_to_bf16_bits(src[i]));
}

__global__ void fill_zero_u32(uint32_t* p, int64_t n) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        p[i] = 0u;
}

static int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

static int check_lmhead(const void* hidden, int64_t n, int64_t h, int64_t ldh, const void* weight, int64_t v, int64_t ldw,
                        const int64_t* targets) {
    if (n < 0 || h <= 0 || v <= 0) return fail(NRL_E_INVALID, "bad shape");
    if (h % 8 || ldh % 8 || ldw % 8) return fail(NRL_E_INVALID, "hidden size and row strides must be multiples of 8");
    if (n > 0 && (!hidden || !weight || !targets)) return fail(NRL_E_INVALID, "null argument");
    if ((reinterpret_cast<uintptr_t>(hidden) & 15) || (reinterpret_cast<uintptr_t>(weight) & 15))
        return fail(NRL_E_INVALID, "hidden and weight must be 16-byte aligned");
    if (ldh < h || ldw < h) return fail(NRL_E_INVALID, "row stride shorter than the hidden size");
    return NRL_OK;
}

}  // namespace nrl

using namespace nrl;

static int fwd_splits(int64_t n, int64_t v) {
    const int64_t row_blocks = (n + GB_M - 1) / GB_M, tiles = (v + GB_N - 1) / GB_N;
    int64_t s = (512 + row_blocks - 1) / row_blocks;  // aim at two workgroups per CU
    if (s > tiles) s = tiles;
    if (s > 64) s = 64;
    return static_cast<int>(s < 1 ? 1 : s);
}

extern "C" int64_t nrl_lmhead_fwd_workspace_bytes(int64_t n_tokens, int64_t vocab) {
    const int64_t n = n_tokens < 1 ? 1 : n_tokens;
    return (2 * fwd_splits(n, vocab) + 1) * n * static_cast<int64_t>(sizeof(float));
}

extern "C" int nrl_lmhead_logprob_fwd(const void* hidden, int64_t n_tokens, int64_t hidden_size, int64_t ldh,
                                      const void* weight, int64_t vocab, int64_t ldw, const int64_t* targets,
                                      int64_t vocab_start, int64_t vocab_end, float* logprob_out, float* lse_out,
                                      void* workspace, int64_t workspace_bytes, void* stream) {
    if (int e = check_lmhead(hidden, n_tokens, hidden_size, ldh, weight, vocab, ldw, targets)) return e;
    if (vocab_end - vocab_start != vocab) return fail(NRL_E_INVALID, "vocab range does not span the rows of W");
    if (n_tokens == 0) return NRL_OK;
    if (!logprob_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (workspace_bytes < nrl_lmhead_fwd_workspace_bytes(n_tokens, vocab)) return fail(NRL_E_WORKSPACE, "workspace too small");
    const int splits = fwd_splits(n_tokens, vocab);
    float* ws = static_cast<float*>(workspace);
    LmFwdArgs a;
    a.op.a = static_cast<const uint16_t*>(hidden); a.op.b = static_cast<const uint16_t*>(weight);
    a.op.lda = ldh; a.op.ldb = ldw; a.op.m = n_tokens; a.op.n = vocab; a.op.k = hidden_size;
    a.targets = targets; a.vocab_start = vocab_start; a.n_splits = splits;
    a.part_m = ws; a.part_s = ws + static_cast<int64_t>(splits) * n_tokens; a.xt = ws + 2 * static_cast<int64_t>(splits) * n_tokens;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t row_blocks = (n_tokens + GB_M - 1) / GB_M;
    if (row_blocks >= (1ll << 31)) return fail(NRL_E_INVALID, "too many tokens");
    fill_zero_u32<<<dim3(256), dim3(256), 0, s>>>(reinterpret_cast<uint32_t*>(a.xt), n_tokens);
    lmhead_fwd_kernel<<<dim3((unsigned)row_blocks, (unsigned)splits), dim3(GB_THREADS), 0, s>>>(a);
    lmhead_fwd_finish_kernel<<<dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, s>>>(
        n_tokens, splits, a.part_m, a.part_s, a.xt, targets, vocab_start, vocab_end, logprob_out, lse_out);
    return check_launch("lmhead_logprob_fwd");
}

static int64_t bwd_chunk(int64_t n) { return n < 4096 ? round_up(n < 1 ? 1 : n, 64) : 4096; }

extern "C" int64_t nrl_lmhead_bwd_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab) {
    const int64_t chunk = bwd_chunk(n_tokens), vp = round_up(vocab, 64);
    int64_t b = 0;
    b += hidden_size * vp * 2;        // W^T
    b += chunk * vp * 2;              // G
    b += vocab * chunk * 2;           // G^T
    b += hidden_size * chunk * 2;     // hidden chunk^T
    b += vocab * hidden_size * 4;     // dW accumulator (fp32)
    return b + 1024;
}

extern "C" int nrl_lmhead_logprob_bwd(const void* hidden, int64_t n_tokens, int64_t hidden_size, int64_t ldh,
                                      const void* weight, int64_t vocab, int64_t ldw, const int64_t* targets,
                                      int64_t vocab_start, int64_t vocab_end, const float* lse, const float* grad,
                                      float* dhidden_out, int64_t ld_dh, void* dweight_out, int64_t ld_dw, void* workspace,
                                      int64_t workspace_bytes, void* stream) {
    if (int e = check_lmhead(hidden, n_tokens, hidden_size, ldh, weight, vocab, ldw, targets)) return e;
    if (vocab_end - vocab_start != vocab) return fail(NRL_E_INVALID, "vocab range does not span the rows of W");
    if (!dweight_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (n_tokens > 0 && (!lse || !grad || !dhidden_out)) return fail(NRL_E_INVALID, "null argument");
    if (workspace_bytes < nrl_lmhead_bwd_workspace_bytes(n_tokens, hidden_size, vocab)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return fail(NRL_E_INVALID, "workspace must be 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t chunk = bwd_chunk(n_tokens), vp = round_up(vocab, 64), h = hidden_size;
    char* ws = static_cast<char*>(workspace);
    uint16_t* wt = reinterpret_cast<uint16_t*>(ws); ws += h * vp * 2;
    uint16_t* g = reinterpret_cast<uint16_t*>(ws); ws += chunk * vp * 2;
    uint16_t* gt = reinterpret_cast<uint16_t*>(ws); ws += vocab * chunk * 2;
    uint16_t* ht = reinterpret_cast<uint16_t*>(ws); ws += h * chunk * 2;
    float* dw = reinterpret_cast<float*>(ws);
    const uint16_t* hid = static_cast<const uint16_t*>(hidden);
    const uint16_t* w = static_cast<const uint16_t*>(weight);

    // W^T [H, vp] (zero-padded columns) and a zeroed fp32 dW accumulator
    transpose_bf16_kernel<<<dim3((unsigned)((h + 63) / 64), (unsigned)((vp + 63) / 64)), dim3(256), 0, s>>>(w, vocab, h, ldw, wt, vp, vp);
    fill_zero_u32<<<dim3(2048), dim3(256), 0, s>>>(reinterpret_cast<uint32_t*>(dw), vocab * h);

    for (int64_t t0 = 0; t0 < n_tokens; t0 += chunk) {
        const int64_t rows = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;
        const int64_t rows_pad = round_up(rows, 64);
        // G / G^T for this chunk
        LmGradArgs ga;
        ga.op.a = hid + t0 * ldh; ga.op.b = w; ga.op.lda = ldh; ga.op.ldb = ldw; ga.op.m = rows; ga.op.n = vocab; ga.op.k = h;
        ga.targets = targets + t0; ga.vocab_start = vocab_start; ga.lse = lse + t0; ga.grad = grad + t0;
        ga.g = g; ga.ldg = vp; ga.gt = gt; ga.ldgt = chunk;
        if (rows_pad < chunk) fill_zero_u32<<<dim3(2048), dim3(256), 0, s>>>(reinterpret_cast<uint32_t*>(gt), vocab * chunk / 2);
        lmhead_grad_kernel<<<dim3((unsigned)((rows + GB_M - 1) / GB_M), (unsigned)((vocab + GB_N - 1) / GB_N)), dim3(GB_THREADS), 0, s>>>(ga);
        // dH[chunk] = G [rows, V] * (W^T [H, V])^T
        GemmOperands dh;
        dh.a = g; dh.lda = vp; dh.b = wt; dh.ldb = vp; dh.m = rows; dh.n = h; dh.k = vp;
        gemm_f32_kernel<false><<<dim3((unsigned)((rows + GB_M - 1) / GB_M), (unsigned)((h + GB_N - 1) / GB_N)), dim3(GB_THREADS), 0, s>>>(
            dh, dhidden_out + t0 * ld_dh, ld_dh);
        // dW += G^T [V, rows] * (hidden^T [H, rows])^T
        transpose_bf16_kernel<<<dim3((unsigned)((h + 63) / 64), (unsigned)((rows_pad + 63) / 64)), dim3(256), 0, s>>>(
            hid + t0 * ldh, rows, h, ldh, ht, chunk, rows_pad);
        GemmOperands dwo;
        dwo.a = gt; dwo.lda = chunk; dwo.b = ht; dwo.ldb = chunk; dwo.m = vocab; dwo.n = h; dwo.k = rows_pad;
        gemm_f32_kernel<true><<<dim3((unsigned)((vocab + GB_M - 1) / GB_M), (unsigned)((h + GB_N - 1) / GB_N)), dim3(GB_THREADS), 0, s>>>(
            dwo, dw, h);
    }
    // narrow dW once
    {
        uint16_t* out = static_cast<uint16_t*>(dweight_out);
        if (ld_dw == h) {
            f32_to_bf16_kernel<<<dim3(2048), dim3(256), 0, s>>>(dw, out, vocab * h);
        } else {
            for (int64_t r = 0; r < vocab; ++r) f32_to_bf16_kernel<<<dim3(4), dim3(256), 0, s>>>(dw + r * h, out + r * ld_dw, h);
        }
    }
    return check_launch("lmhead_logprob_bwd");
}

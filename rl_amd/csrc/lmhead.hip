// K6: fused lm_head -> token logprob (hidden @ W^T, never materialising the full logits) and its
// backward (dH, dW), on the gfx950 matrix cores.
//
// Three bf16 MFMA GEMM cores, C[M,N] = A[M,K] * B[N,K]^T with fp32 accumulation (v_mfma_f32_32x32x16_bf16,
// 4 wave64, one per SIMD, 256 accumulator registers each), serve every product:
//   * core B (K a multiple of 64; forward and recomputing gradient): 256 x 256 tile, waves 2 x 2 with 128 x 128
//     each, both operands double-buffered in LDS by direct global-to-LDS loads;
//   * core C (K a multiple of 64; the backward's dH and dW products): 256 x 256 tile, waves side by side with
//     256 x 64 each, operand A through LDS, operand B from a fragment-major copy straight into registers;
//   * core A, the general one (K a multiple of 8): 256 x 128 tile, operands staged through registers
//     into one padded LDS buffer.
// Workgroups are numbered so that the 32 that share an XCD (and its L2) cover a 4 x 8 patch of tiles.
// Epilogues:
//   LSE    forward, computed as logits^T = W hidden^T so that the vocabulary runs along the accumulator
//          rows a lane owns: the tile's logits are rounded to bf16 (the reference's matmul returns
//          bf16) and folded into a running (max, sum-exp) per token column without any cross-lane
//          traffic while the workgroup walks its vocabulary tiles; the target's logit is captured on the
//          way.  Only [tokens] sized partials leave the chip.
//   GRAD   backward: recomputed tile -> the softmax part -g * exp(x - lse) of the logits' gradient, written as
//          bf16 row-major (for dH = G W) and, with the one-hot term g at the target added, transposed (for
//          dW = G^T hidden), for one token chunk at a time.  The one-hot term of dH, g * W[target], is added
//          in fp32 by its own kernel: it is the one large element of a row of G, and narrowing it to bf16
//          would put its rounding error (up to 2^-8, coherent over the row) straight into dH.
//   STORE / ACCUM  plain fp32 C = or C += for dH and dW.
// The vocabulary is walked in tiles while the token chunk bounds what is materialised:
// chunk x V bf16 for G and G^T (5 GB each at chunk 16384, V 151936) instead of N x V.

#include <float.h>
#include <stdlib.h>
#include <type_traits>
#include <math.h>

#include "common.hpp"

namespace nrl {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GB_THREADS = 256;  // 4 wave64, whatever the core

struct GemmOperands {
    const uint16_t* a;  // [M, K] row stride lda
    const uint16_t* b;  // [N, K] row stride ldb
    int64_t lda, ldb, m, n, k;  // k multiple of 8; slabs beyond k read as zero
    // An extent that only the device knows (the number of tokens that carry a gradient): when `live` is set, the
    // kernel replaces m (live_dim 1) or k (live_dim 2, rounded up to 64) by clamp(live[0] - live_from, 0, that
    // extent) before it starts, and leaves at once when nothing is left.
    const int32_t* live = nullptr;
    int64_t live_from = 0;
    int live_dim = 0;
};

// applies the device-side extent; false when the product is empty
__device__ __forceinline__ bool resolve_live(GemmOperands& op) {
    if (op.live) {
        int64_t r = static_cast<int64_t>(op.live[0]) - op.live_from;
        r = r < 0 ? 0 : r;
        if (op.live_dim == 1) op.m = r < op.m ? r : op.m;
        else { r = (r + 63) / 64 * 64; op.k = r < op.k ? r : op.k; }
    }
    return op.m > 0 && op.k > 0 && op.n > 0;
}

// accumulator element e (0..15) of lane l in a 32x32 tile: column l % 32, row 8*(e/4) + 4*(l/32) + e%4
__device__ __forceinline__ int acc_row(int e, int lane) { return 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3); }

// ---------------------------------------------------------------------------------------------
// Core A: 256 x 128 tile (wave tile 128 x 64), any K multiple of 8.  Slab k+1 travels through
// registers while slab k is consumed from one padded LDS buffer (row stride 72 elements).
// ---------------------------------------------------------------------------------------------
struct CoreA {
    static constexpr int BM = 256, BN = 128, NI = 4, NJ = 2, BK = 64, LD = BK + 8, WAVES_N = 2;
    static constexpr int LDS_BYTES = (BM + BN) * LD * 2;
    static constexpr int A_LOADS = BM * BK / 8 / GB_THREADS, B_LOADS = BN * BK / 8 / GB_THREADS;
    struct Regs {
        u32x4 a[A_LOADS];
        u32x4 b[B_LOADS];
    };

    __device__ static __forceinline__ void load_slab(const GemmOperands& op, int64_t row0, int64_t col0, int64_t k0, Regs& r) {
        const int tid = threadIdx.x;
        const u32x4 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) {
            const int c = tid + GB_THREADS * j;
            const int rr = c >> 3, kc = c & 7;
            int64_t grow = row0 + rr;
            grow = grow < op.m ? grow : op.m - 1;
            const int64_t kk = k0 + kc * 8;
            r.a[j] = kk < op.k ? *reinterpret_cast<const u32x4*>(op.a + grow * op.lda + kk) : zero;
        }
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            const int c = tid + GB_THREADS * j;
            const int rr = c >> 3, kc = c & 7;
            int64_t grow = col0 + rr;
            grow = grow < op.n ? grow : op.n - 1;
            const int64_t kk = k0 + kc * 8;
            r.b[j] = kk < op.k ? *reinterpret_cast<const u32x4*>(op.b + grow * op.ldb + kk) : zero;
        }
    }

    __device__ static __forceinline__ void store_slab(const Regs& r, uint16_t* As, uint16_t* Bs) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) {
            const int c = tid + GB_THREADS * j;
            *reinterpret_cast<u32x4*>(As + (c >> 3) * LD + (c & 7) * 8) = r.a[j];
        }
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            const int c = tid + GB_THREADS * j;
            *reinterpret_cast<u32x4*>(Bs + (c >> 3) * LD + (c & 7) * 8) = r.b[j];
        }
    }

    // acc[i][j] += A[row0.., :] * B[col0.., :]^T for the workgroup's tile
    __device__ static __forceinline__ void tile(const GemmOperands& op, int64_t row0, int64_t col0, f32x16 (&acc)[NI][NJ],
                                                unsigned char* lds) {
        uint16_t* As = reinterpret_cast<uint16_t*>(lds);
        uint16_t* Bs = As + BM * LD;
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
        const int wm = wave >> 1, wn = wave & 1;
        const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
        Regs regs;
        const int64_t nk = (op.k + BK - 1) / BK;
        load_slab(op, row0, col0, 0, regs);
        __syncthreads();  // previous users of the LDS tiles are done
        store_slab(regs, As, Bs);
        __syncthreads();
        for (int64_t kt = 0; kt < nk; ++kt) {
            if (kt + 1 < nk) load_slab(op, row0, col0, (kt + 1) * BK, regs);
#pragma unroll
            for (int ks = 0; ks < BK / 16; ++ks) {
                bf16x8 af[NI], bfr[NJ];
#pragma unroll
                for (int i = 0; i < NI; ++i)
                    af[i] = *reinterpret_cast<const bf16x8*>(As + (wm * 128 + i * 32 + frag_row) * LD + ks * 16 + frag_k);
#pragma unroll
                for (int j = 0; j < NJ; ++j)
                    bfr[j] = *reinterpret_cast<const bf16x8*>(Bs + (wn * 64 + j * 32 + frag_row) * LD + ks * 16 + frag_k);
#pragma unroll
                for (int i = 0; i < NI; ++i)
#pragma unroll
                    for (int j = 0; j < NJ; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
            }
            __syncthreads();
            if (kt + 1 < nk) {
                store_slab(regs, As, Bs);
                __syncthreads();
            }
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Core B: 256 x 256 tile (wave tile 128 x 128: 16 MFMA tiles, 256 accumulator registers, one wave per
// SIMD), K a multiple of 64.  Two LDS buffers per operand (4 x 32 KiB); slabs k+1 and k+2 are fetched by direct
// global-to-LDS loads while slab k is consumed, one barrier per slab.  A 64-element row is 8 chunks
// of 16 bytes; chunk c of row r sits at chunk position c ^ ((r >> 1) & 7), which keeps the rows unpadded
// (a wave's direct load fills 1 KiB contiguously) and the wave's 16-byte fragment reads (32 rows x 2
// chunks) free of bank conflicts: measured 8.7 cycles per ds_read_b128, the same as a contiguous read,
// against 12.6 with the key r & 7 and 32 without swizzling.  Per 16-wide k step a wave issues 8 fragment reads for 16 MFMAs.
// ---------------------------------------------------------------------------------------------
struct CoreB {
    static constexpr int BM = 256, BN = 256, NI = 4, NJ = 4, BK = 64, WAVES_N = 2;
    static constexpr int TILE_BYTES = 256 * BK * 2;  // one operand, one buffer
    static constexpr int LDS_BYTES = 4 * TILE_BYTES;  // A0 A1 B0 B1
    static constexpr int ROUNDS = 256 * BK / 8 / GB_THREADS;  // direct loads per lane, operand and slab: 8

    struct Ctx {
        const char* pa;  // first row of the tile, bytes
        const char* pb;
        uint32_t voa[ROUNDS], vob[ROUNDS];  // lane's source offset in each round (rows past the end clamped)
        uint32_t aoff[BK / 16], boff[BK / 16];  // lane's fragment address in LDS for each k step (buffer 0, tile 0)
        int wave;                               // wave index, held in a scalar register
    };

    // direct load number d (0..7: operand A rounds, 8..15: operand B rounds) of slab k0 into buffer buf
    __device__ static __forceinline__ void issue_one(const Ctx& c, unsigned char* lds, int buf, int64_t k0, int d) {
        const int op = d / ROUNDS, j = d % ROUNDS;
        unsigned char* dst = lds + (2 * op + buf) * TILE_BYTES + (j * GB_THREADS + c.wave * 64) * 16;
        const char* src = (op ? c.pb : c.pa) + k0 * 2 + (op ? c.vob[j] : c.voa[j]);
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const __attribute__((address_space(1))) void*>(reinterpret_cast<uintptr_t>(src)),
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    }
    __device__ static __forceinline__ void issue(const Ctx& c, unsigned char* lds, int buf, int64_t k0) {
#pragma unroll
        for (int d = 0; d < 2 * ROUNDS; ++d) issue_one(c, lds, buf, k0, d);
    }

    // Fragment reads are written as inline assembly.  A read the compiler can see is treated as possibly
    // aliasing every direct-to-LDS load still in flight and gets a vmcnt(0) in front of it, which stalls the
    // wave for a full memory latency in the middle of the slab; the two never touch the same buffer here
    // (the slab barrier orders them), so the reads are hidden from that analysis and waited for by hand.
    __device__ static __forceinline__ bf16x8 lds_read16(uint32_t addr, int imm) {
        bf16x8 v;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(imm));
        return v;
    }
    // every LDS read issued so far has returned; the operands tie the wait to the fragments it guards
    __device__ static __forceinline__ void wait_frags(bf16x8 (&a)[NI], bf16x8 (&b)[NJ]) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
    }

    static constexpr int KS = BK / 16;
    static constexpr int LATE = ROUNDS;  // of a slab's 16 direct loads, those issued during the following slab's first k step

    // One slab out of buffer BUF with one wave per SIMD: nothing else hides latencies, so the order is fixed by
    // hand.  On entry the fragments of the slab's k step 0 are in flight into set 0; on exit those of the next
    // slab (buffer BUF ^ 1) are.  The fragments of the last k step are in registers once that step starts, so
    // from there on this wave no longer reads BUF: the wait for the other buffer's direct loads and the workgroup
    // barrier sit at the start of the last step, no LDS latency is exposed between two slabs, and the freed
    // buffer starts filling at once with the slab after the next (k_load): half of its 16 direct loads go out
    // behind every second MFMA of this last step, the other half (k_late, into BUF ^ 1 as seen from the next
    // slab) behind every second MFMA of the next slab's first step.  Measured against all 16 in one step, or 4 /
    // 2 early: this split was fastest on every shape.  The 8 fragment reads of k step ks + 1 follow the first 8
    // MFMAs of step ks.
    template <int BUF>
    __device__ static __forceinline__ void compute(const Ctx& c, unsigned char* lds, f32x16 (&acc)[NI][NJ],
                                                   bf16x8 (&af)[2][NI], bf16x8 (&bfr)[2][NJ], int64_t k_load, int64_t k_late) {
        auto frag_one = [&](int buf, int ks, int set, int f) {
            if (f < NI) af[set][f] = lds_read16(c.aoff[ks], buf * TILE_BYTES + f * 32 * BK * 2);
            else bfr[set][f - NI] = lds_read16(c.boff[ks], buf * TILE_BYTES + (f - NI) * 32 * BK * 2);
        };
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            wait_frags(af[ks & 1], bfr[ks & 1]);
            if (ks == KS - 1) {
                // this wave is done reading BUF; the other buffer's loads (issued during the previous slab's
                // last step and this slab's first steps) must have landed before anyone reads it
                asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int idx = i * NJ + j;
                    __builtin_amdgcn_sched_barrier(0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], bfr[ks & 1][j], acc[i][j], 0, 0, 0);
                    constexpr int EARLY = 2 * ROUNDS - LATE, GAP = NI * NJ / EARLY;
                    if (ks == KS - 1 && idx % GAP == 0) {
                        // the freed buffer takes the slab after the next: direct loads behind this step's MFMAs
                        __builtin_amdgcn_sched_barrier(0);
                        issue_one(c, lds, BUF, k_load, idx / GAP);
                    }
                    const int n = ks * NI * NJ + idx;
                    if (n % 2 == 0 && n / 2 < LATE) {
                        // ... and the rest of the slab that the previous slab started loading into the other buffer
                        __builtin_amdgcn_sched_barrier(0);
                        issue_one(c, lds, BUF ^ 1, k_late, EARLY + n / 2);
                    }
                    if (idx < NI + NJ) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (ks + 1 < KS) frag_one(BUF, ks + 1, (ks + 1) & 1, idx);
                        else frag_one(BUF ^ 1, 0, 0, idx);
                    }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    __device__ static __forceinline__ void tile(const GemmOperands& op, int64_t row0, int64_t col0, f32x16 (&acc)[NI][NJ],
                                                unsigned char* lds) {
        static_assert(NI + NJ <= NI * NJ && 2 * ROUNDS == NI * NJ, "one direct load behind each MFMA of a k step");
        static_assert(LATE >= 0 && LATE < 2 * ROUNDS && (NI * NJ) % (2 * ROUNDS - LATE) == 0 && LATE <= 3 * NI * NJ / 2, "load schedule");
        // (an opaque copy of the thread index: everything derived from it below is recomputed per tile, about a
        // hundred instructions, instead of being hoisted out of the caller's tile loop and kept in registers, or
        // spilled, across its epilogue)
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int wm = wave >> 1, wn = wave & 1;
        Ctx c;
        c.wave = wave;
        c.pa = reinterpret_cast<const char*>(op.a + row0 * op.lda);
        c.pb = reinterpret_cast<const char*>(op.b + col0 * op.ldb);
        const int lr = tid >> 3, cg = (tid & 7) ^ ((lr >> 1) & 7);
        const int last_a = static_cast<int>(op.m - 1 - row0 < 255 ? op.m - 1 - row0 : 255);
        const int last_b = static_cast<int>(op.n - 1 - col0 < 255 ? op.n - 1 - col0 : 255);
#pragma unroll
        for (int j = 0; j < ROUNDS; ++j) {
            const int r = j * 32 + lr;
            c.voa[j] = static_cast<uint32_t>((r < last_a ? r : last_a) * op.lda + cg * 8) * 2u;
            c.vob[j] = static_cast<uint32_t>((r < last_b ? r : last_b) * op.ldb + cg * 8) * 2u;
        }
        const int fr = lane & 31, fh = lane >> 5;
        const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint32_t sw = static_cast<uint32_t>(((ks * 2 + fh) ^ ((fr >> 1) & 7)) * 16);
            c.aoff[ks] = lds_base + static_cast<uint32_t>((wm * 128 + fr) * BK * 2) + sw;
            c.boff[ks] = lds_base + static_cast<uint32_t>(2 * TILE_BYTES + (wn * 128 + fr) * BK * 2) + sw;
        }
        const int64_t nk = op.k / BK;
        const int64_t k_last = (nk - 1) * BK;
        auto slab_k = [&](int64_t kt) { return kt < nk ? kt * BK : k_last; };  // past the end: the last slab again, unused
        // every wave has passed the barrier inside the previous tile's last slab and has since only read
        // registers, so both buffers are free: slab 0 and slab 1 start now
        issue(c, lds, 0, 0);
#pragma unroll
        for (int d = 0; d < 2 * ROUNDS - LATE; ++d) issue_one(c, lds, 1, slab_k(1), d);
        // slab 0 has landed everywhere
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * ROUNDS - LATE) : "memory");
        bf16x8 af[2][NI], bfr[2][NJ];
#pragma unroll
        for (int f = 0; f < NI + NJ; ++f) {
            if (f < NI) af[0][f] = lds_read16(c.aoff[0], f * 32 * BK * 2);
            else bfr[0][f - NI] = lds_read16(c.boff[0], (f - NI) * 32 * BK * 2);
        }
        int64_t kt = 0;
        for (; kt + 1 < nk; kt += 2) {
            compute<0>(c, lds, acc, af, bfr, slab_k(kt + 2), slab_k(kt + 1));
            compute<1>(c, lds, acc, af, bfr, slab_k(kt + 3), slab_k(kt + 2));
        }
        if (kt < nk) compute<0>(c, lds, acc, af, bfr, k_last, k_last);
        // The last slab read ahead into fragments nobody uses.  Their registers must stay allocated until the
        // reads have returned: the compiler takes an asm output for complete at once, and a register it hands
        // out again (a load address, say) would be overwritten when the LDS data arrives.
        wait_frags(af[0], bfr[0]);
        // likewise the direct loads the last slab issued (copies of itself, never read) must not outlive the tile
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    }
};

// ---------------------------------------------------------------------------------------------
// Core C: 256 x 256 tile, the four waves side by side along N (wave tile 256 x 64: NI = 8, NJ = 2), K a multiple
// of 64.  Only operand A goes through LDS (four 32 KiB buffers filled by direct global-to-LDS loads, three slabs
// ahead); each wave reads its own operand-B fragments straight from memory into registers, one slab ahead.  For
// that B is stored "fragment-major": the 1 KiB that the 64 lanes of a wave feed to one matrix instruction (32 rows
// x 16 k) is contiguous, lane by lane, and the blocks of a 32-row group follow each other along k -- a wave's load
// of a fragment is then one fully used 1 KiB burst.  Per 16-wide k step a wave issues 8 LDS fragment reads for 16
// MFMAs like core B, but the workgroup writes half as much into LDS and no wave reads B from it.
//   element (n, k) of B sits at ((n / 32 * K16 + k / 16) * 64 + n % 32 + 32 * (k % 16 / 8)) * 8 + k % 8,
//   K16 = ldb / 16 (ldb: the allocated k extent, a multiple of 64); row groups are allocated up to a multiple of 256 rows.
// ---------------------------------------------------------------------------------------------
template <int SPREAD> struct CoreCT {
    static constexpr int BM = 256, BN = 256, NI = 8, NJ = 2, BK = 64, WAVES_N = 4;
    static constexpr int KS = BK / 16;
    static constexpr int NBUF = 4;
    static constexpr int TILE_BYTES = 256 * BK * 2;
    static constexpr int LDS_BYTES = NBUF * TILE_BYTES;
    static constexpr int ROUNDS = 256 * BK / 8 / GB_THREADS;  // 8 direct loads per lane and slab

    struct Ctx {
        const char* pa;
        uint32_t voa[ROUNDS];
        uint32_t aoff[2][KS];   // lane's fragment address for each k step: buffers 0/1 and buffers 2/3 (tile row group 0)
        uint64_t pb[NJ];        // this wave's two row groups of B at k = 0 (uniform)
        uint32_t vlane;         // lane * 16
        int wave;
    };

    __device__ static __forceinline__ void issue_a(const Ctx& c, unsigned char* lds, int buf, int64_t k0, int j) {
        unsigned char* dst = lds + buf * TILE_BYTES + (j * GB_THREADS + c.wave * 64) * 16;
        const char* src = c.pa + k0 * 2 + c.voa[j];
        __builtin_amdgcn_global_load_lds(reinterpret_cast<const __attribute__((address_space(1))) void*>(reinterpret_cast<uintptr_t>(src)),
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    }
    // fragment (k step ks, row group j) of the slab that starts at k0
    template <int KSTEP>
    __device__ static __forceinline__ bf16x8 load_b(const Ctx& c, int64_t k0, int j) {
        bf16x8 v;
        const uint64_t base = c.pb[j] + static_cast<uint64_t>(k0) * 64;  // k0 / 16 blocks of 1 KiB
        asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(v) : "v"(c.vlane), "s"(base), "n"(KSTEP * 1024));
        return v;
    }
    __device__ static __forceinline__ bf16x8 lds_read16(uint32_t addr, int imm) {
        bf16x8 v;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(imm));
        return v;
    }
    __device__ static __forceinline__ void wait_a(bf16x8 (&a)[NI]) {
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]));
    }
    template <int N> __device__ static __forceinline__ void wait_b(bf16x8 (&b)[KS][NJ]) {
        asm volatile("s_waitcnt vmcnt(%8)"
                     : "+v"(b[0][0]), "+v"(b[0][1]), "+v"(b[1][0]), "+v"(b[1][1]), "+v"(b[2][0]), "+v"(b[2][1]), "+v"(b[3][0]), "+v"(b[3][1])
                     : "n"(N));
    }

    static constexpr int LEAD = 2 * KS - 1;  // B fragments are fetched this many k steps ahead
    static_assert(NI == 8 && NJ == 2 && KS == 4 && ROUNDS == 2 * KS, "the waits below list their registers and count the operations of a k step");

    // fragments of k step `ks` (0 .. 2 KS - 1, counted from the slab that starts at k0) -> the ring of 2 KS register pairs
    __device__ static __forceinline__ void fetch_b(const Ctx& c, bf16x8 (&bfr)[2][KS][NJ], int set, int ks, int64_t k0, int j) {
        if (ks == 0) bfr[set][0][j] = load_b<0>(c, k0, j);
        if (ks == 1) bfr[set][1][j] = load_b<1>(c, k0, j);
        if (ks == 2) bfr[set][2][j] = load_b<2>(c, k0, j);
        if (ks == 3) bfr[set][3][j] = load_b<3>(c, k0, j);
    }

    // One slab out of LDS buffer SLOT; its B fragments are in register set SLOT & 1 of a ring of 2 KS k steps.  On
    // entry the A fragments of k step 0 are in flight into af[0].  Every k step issues four vector-memory operations,
    // behind its first MFMAs: the two B fragments of the k step LEAD steps ahead (into the registers that the k
    // step before this one has just finished with), then two of the eight direct loads of the slab three ahead
    // (into the buffer that the previous slab's barrier freed).  Memory operations complete in order, so at the
    // start of a k step "all but the youngest 4 (LEAD - 1) + 2" says that its B fragments are there.  At the start
    // of the last k step this wave holds every fragment it needs from SLOT; the next slab's direct loads were
    // issued two slabs ago or, for a tile's second slab, up to 20 operations before this point, hence vmcnt(20),
    // and the barrier frees SLOT for the slab four ahead.
    template <int SLOT>
    __device__ static __forceinline__ void compute(const Ctx& c, unsigned char* lds, f32x16 (&acc)[NI][NJ], bf16x8 (&af)[2][NI],
                                                   bf16x8 (&bfr)[2][KS][NJ], int64_t k_b1, int64_t k_b2, int64_t k_a) {
        constexpr int SET = SLOT & 1, NEXT = (SLOT + 1) % NBUF;
        auto frag_a = [&](int slot, int ks, int set, int f) {
            af[set][f] = lds_read16(c.aoff[slot >> 1][ks], (slot & 1) * TILE_BYTES + f * 32 * BK * 2);
        };
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            wait_a(af[ks & 1]);
            if (ks == KS - 1) {
                wait_b<20>(bfr[SET]);
                asm volatile("s_barrier" ::: "memory");
            } else {
                wait_b<4 * (LEAD - 1) + 2>(bfr[SET]);
            }
#pragma unroll
            for (int i = 0; i < NI; ++i) {
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int idx = i * NJ + j;
                    __builtin_amdgcn_sched_barrier(0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], bfr[SET][ks][j], acc[i][j], 0, 0, 0);
                    if (idx == 0 || idx == SPREAD) {
                        __builtin_amdgcn_sched_barrier(0);
                        // k step ks + LEAD: ks == 0 -> next slab's last k step, otherwise the slab after it
                        if (ks == 0) fetch_b(c, bfr, SET ^ 1, KS - 1, k_b1, idx / SPREAD);
                        else fetch_b(c, bfr, SET, ks - 1, k_b2, idx / SPREAD);
                    }
                    if (idx == 2 * SPREAD || idx == 3 * SPREAD) {
                        __builtin_amdgcn_sched_barrier(0);
                        issue_a(c, lds, (SLOT + 3) % NBUF, k_a, ks * 2 + idx / SPREAD - 2);
                    }
                    if (idx < NI) {
                        __builtin_amdgcn_sched_barrier(0);
                        if (ks + 1 < KS) frag_a(SLOT, ks + 1, (ks + 1) & 1, idx);
                        else frag_a(NEXT, 0, 0, idx);
                    }
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }

    __device__ static __forceinline__ void tile(const GemmOperands& op, int64_t row0, int64_t col0, f32x16 (&acc)[NI][NJ],
                                                unsigned char* lds) {
        int tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
        Ctx c;
        c.wave = wave;
        c.vlane = static_cast<uint32_t>(lane * 16);
        c.pa = reinterpret_cast<const char*>(op.a + row0 * op.lda);
        const int64_t k16 = op.ldb / 16;
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            c.pb[j] = reinterpret_cast<uint64_t>(op.b) + static_cast<uint64_t>(((col0 >> 5) + wave * NJ + j) * k16) * 1024u;
        const int lr = tid >> 3, cg = (tid & 7) ^ ((lr >> 1) & 7);
        const int last_a = static_cast<int>(op.m - 1 - row0 < 255 ? op.m - 1 - row0 : 255);
#pragma unroll
        for (int j = 0; j < ROUNDS; ++j) {
            const int r = j * 32 + lr;
            c.voa[j] = static_cast<uint32_t>((r < last_a ? r : last_a) * op.lda + cg * 8) * 2u;
        }
        const int fr = lane & 31, fh = lane >> 5;
        const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint32_t sw = static_cast<uint32_t>(((ks * 2 + fh) ^ ((fr >> 1) & 7)) * 16);
            c.aoff[0][ks] = lds_base + static_cast<uint32_t>(fr * BK * 2) + sw;
            c.aoff[1][ks] = c.aoff[0][ks] + 2 * TILE_BYTES;
        }
        const int64_t nk = op.k / BK;
        const int64_t k_last = (nk - 1) * BK;
        auto slab_k = [&](int64_t kt) { return kt < nk ? kt * BK : k_last; };
        bf16x8 af[2][NI], bfr[2][KS][NJ];
        // order: the B fragments of the first LEAD k steps, then slabs 0, 1, 2 of A (the waits count on it)
#pragma unroll
        for (int g = 0; g < LEAD; ++g)
#pragma unroll
            for (int j = 0; j < NJ; ++j) fetch_b(c, bfr, g / KS, g % KS, g < KS ? 0 : slab_k(1), j);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < ROUNDS; ++j) issue_a(c, lds, 0, 0, j);
#pragma unroll
        for (int j = 0; j < ROUNDS; ++j) issue_a(c, lds, 1, slab_k(1), j);
#pragma unroll
        for (int j = 0; j < ROUNDS; ++j) issue_a(c, lds, 2, slab_k(2), j);
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * ROUNDS) : "memory");  // slab 0 of A has landed everywhere
#pragma unroll
        for (int f = 0; f < NI; ++f) af[0][f] = lds_read16(c.aoff[0][0], f * 32 * BK * 2);
        int64_t kt = 0;
        for (; kt + 3 < nk; kt += 4) {
            compute<0>(c, lds, acc, af, bfr, slab_k(kt + 1), slab_k(kt + 2), slab_k(kt + 3));
            compute<1>(c, lds, acc, af, bfr, slab_k(kt + 2), slab_k(kt + 3), slab_k(kt + 4));
            compute<2>(c, lds, acc, af, bfr, slab_k(kt + 3), slab_k(kt + 4), slab_k(kt + 5));
            compute<3>(c, lds, acc, af, bfr, slab_k(kt + 4), slab_k(kt + 5), slab_k(kt + 6));
        }
        if (kt < nk) compute<0>(c, lds, acc, af, bfr, slab_k(kt + 1), slab_k(kt + 2), slab_k(kt + 3));
        if (kt + 1 < nk) compute<1>(c, lds, acc, af, bfr, slab_k(kt + 2), slab_k(kt + 3), slab_k(kt + 4));
        if (kt + 2 < nk) compute<2>(c, lds, acc, af, bfr, slab_k(kt + 3), slab_k(kt + 4), slab_k(kt + 5));
        // what the last slabs fetched ahead is never used, but its registers and buffers must stay untouched until it
        // has arrived
        wait_a(af[0]);
        wait_b<0>(bfr[0]);
        wait_b<0>(bfr[1]);
        asm volatile("s_barrier" ::: "memory");
    }
};

using CoreC = CoreCT<2>;

template <class Core> __device__ __forceinline__ void zero_acc(f32x16 (&acc)[Core::NI][Core::NJ]) {
#pragma unroll
    for (int i = 0; i < Core::NI; ++i)
#pragma unroll
        for (int j = 0; j < Core::NJ; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
}

// One accumulator element, moved from its accumulation register when it is used: read this way the epilogue takes
// the values block by block, where plain uses let the compiler copy all 256 to vector registers first and spill.
__device__ __forceinline__ float acc_read(float a) {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}

__device__ __forceinline__ float round_bf16(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }

// Tile coordinates of workgroup w of a 1-D launch over an nbx x nby tile grid.  Workgroups go to the
// 8 XCDs (each with its own L2) round-robin by index, so index w runs on XCD w % 8 as that XCD's
// (w / 8)-th workgroup; an XCD's 32 compute units hold one PX x PY patch of tiles at a time (4 x 8 unless said
// otherwise), which share PX A panels and PY B panels through that L2.  Patches past the grid yield false.
template <int PX = 4>
__device__ __forceinline__ bool patch_tile(uint32_t w, int64_t nbx, int64_t nby, int64_t& bx, int64_t& by) {
    constexpr uint32_t PY = 32 / PX;
    static_assert(PX * PY == 32, "a patch is what one XCD holds");
    const uint32_t xcd = w & 7, s = w >> 3;
    const uint32_t patch = (s >> 5) * 8 + xcd, t = s & 31;
    const uint32_t ppy = static_cast<uint32_t>((nby + PY - 1) / PY);  // patches along y
    const uint32_t px = patch / ppy, py = patch - px * ppy;
    // the division runs on the vector unit; hand the (uniform) results back to scalar registers
    bx = __builtin_amdgcn_readfirstlane(static_cast<int>(px * PX + t / PY));
    by = __builtin_amdgcn_readfirstlane(static_cast<int>(py * PY + t % PY));
    return bx < nbx && by < nby;
}
static int64_t patch_grid(int64_t nbx, int64_t nby, int64_t px = 4) {
    const int64_t py = 32 / px, patches = ((nbx + px - 1) / px) * ((nby + py - 1) / py);
    return (patches + 7) / 8 * 8 * 32;
}

// ---------------------------------------------------------------------------------------------
// forward: running log-sum-exp over the vocabulary tiles of one split
// ---------------------------------------------------------------------------------------------
// The product is taken as logits^T = W hidden^T: in the 32 x 32 accumulator tile a lane owns one column
// and 16 rows, so with the vocabulary along the rows the whole log-sum-exp reduction of a tile stays
// inside the lane (NJ token columns per lane, 2 registers of running state each) and no cross-lane
// traffic happens until the very end.
// Kept logits are stored as the forward's accumulators hold them, block by block: a block is 32 vocabulary ids x 32
// tokens, 2 KiB, laid out [half p][lane][8 bf16] with lane = 32 h + token % 32, and the lane's 8 values of half p are
// the ids 16 p + 8 q + 4 h + e of the block (q = 0, 1; e = 0..3), in that order.  Blocks follow each other along the
// vocabulary (ceil(V / 32) of them), then along the tokens (ceil(N / 32)).  The forward writes a block with two
// 1 KiB stores per wave and no shuffle; the backward reads 16 bytes per token and half and regroups in registers.
// Ids past V and tokens past N of the last blocks hold unspecified values.
__host__ __device__ __forceinline__ int64_t kept_block(int64_t token_block, int64_t vocab_block, int64_t n_vb) {
    return (token_block * n_vb + vocab_block) * 2048;
}
static int64_t kept_logits_bytes(int64_t n_tokens, int64_t vocab) {
    return kept_block((n_tokens + 31) / 32, 0, (vocab + 31) / 32);
}

struct LmFwdArgs {
    GemmOperands op;           // a = W [V,H] (m = V), b = hidden [N,H] (n = N)
    const int64_t* targets;    // [N]
    int64_t vocab_start;       // target ids are global; rows of W are local
    int n_splits;
    float* part_m;             // [n_splits, N]
    float* part_s;             // [n_splits, N]
    float* xt;                 // [N] target logit (written by the tile that holds it)
    unsigned char* logits;     // bf16 logits kept for the backward in the block layout (kept_block), or NULL
    int64_t n_vb;              // its vocabulary blocks per token block: ceil(V / 32)
    unsigned int* arrive;      // one zeroed counter per XCD patch of workgroups, or NULL: see patch_cross
    unsigned align_every;      // the patch re-aligns before every align_every-th tile
    unsigned align_spins;      // polls after which a workgroup stops waiting for its patch
};

// The 32 workgroups of an XCD patch share their operand panels through that XCD's L2 only while they read the same
// slab at about the same time; over a walk of 74 vocabulary tiles they drift apart and every panel is then filled
// once per reader.  Before a tile, every workgroup of the patch adds itself to the patch's counter and waits until
// all have (`target` arrivals in total); by default once, before the first tile (fwd_align_every).  The wait is
// bounded: a workgroup that has not seen the others after
// kAlignSpins polls (they may not all be resident, e.g. next to another kernel) opens the counter for good, and the
// patch walks on unaligned, which costs bandwidth, not correctness.
// (512 polls, well under a millisecond, align as well as 4096 did -- 58.7 M KiB of fills against 58.6 M; 64 do not:
// 64.5 M -- and bound what a patch can lose when its workgroups cannot all be resident)
constexpr unsigned kAlignSpins = 512;
constexpr unsigned kAlignOpen = 1u << 24;  // added by a workgroup that gives up: every later target is below it
__device__ __forceinline__ void patch_cross(unsigned int* ctr, unsigned target, unsigned max_spins) {
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned spins = 0;
        while (__hip_atomic_load(ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
            if (++spins > max_spins) {
                __hip_atomic_fetch_add(ctr, kAlignOpen, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(2);
        }
    }
    __syncthreads();
}

// Token tiles per XCD patch of the forward (the other side of the patch counts vocabulary splits).  Without the
// logits 8 token tiles x 4 splits measured 4 % faster than 4 x 8 (58.9 against 61.3 ms at 65536 tokens, V 151936);
// with the logits written it measured 1 % slower, and 16 x 2 and 32 x 1 slower either way.
constexpr int fwd_patch_tokens(bool save) { return save ? 4 : 8; }

template <class Core, bool SAVE>
__global__ __launch_bounds__(GB_THREADS) void lmhead_fwd_kernel(LmFwdArgs a) {
    constexpr int NI = Core::NI, NJ = Core::NJ, BV = Core::BM, BT = Core::BN;  // vocabulary rows x token columns
    __shared__ __attribute__((aligned(1024))) unsigned char lds[Core::LDS_BYTES];
    __shared__ float comb_m[2][BT], comb_s[2][BT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    int64_t bx, by;
    if (!patch_tile<fwd_patch_tokens(SAVE)>(blockIdx.x, (a.op.n + BT - 1) / BT, a.n_splits, bx, by)) return;
    const int64_t tok0 = bx * BT;
    const int split = static_cast<int>(by);
    const int64_t n_tiles = (a.op.m + BV - 1) / BV;
    // (local) target row of each of the tile's token columns, -1 where there is none; kept in LDS so that the
    // registers it would occupy through the K loop stay free
    __shared__ int tgt_s[BT];
    static_assert(BT <= GB_THREADS, "one thread per token column fills the target table");
    if (tid < BT) {
        int64_t t = -1;
        if (tok0 + tid < a.op.n) t = a.targets[tok0 + tid] - a.vocab_start;
        tgt_s[tid] = (t >= 0 && t < a.op.m) ? static_cast<int>(t) : -1;
    }
    __syncthreads();
    // Running (max, sum exp) of the lane's NJ token columns.  They live in LDS, not in registers: the K loop of a
    // tile takes every vector register, and a value that is live across it would be spilled to scratch.  For the
    // same reason everything derived from the thread index is derived again, from an opaque copy, after the K loop.
    __shared__ float run_m_s[NJ][GB_THREADS], run_s_s[NJ][GB_THREADS];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { run_m_s[j][tid] = -1e30f; run_s_s[j][tid] = 0.f; }

    // alignment of the patch (see patch_cross): the workgroups of this patch that exist, and the tiles all of them walk
    unsigned members = 0, common = 0, epoch = 0;
    unsigned int* arrive = nullptr;
    if (a.arrive) {
        constexpr int PX = fwd_patch_tokens(SAVE), PY = 32 / PX;
        const int64_t nbx = (a.op.n + BT - 1) / BT, nby = a.n_splits;
        const int64_t px0 = bx / PX * PX, py0 = by / PY * PY;
        const int64_t cx = nbx - px0 < PX ? nbx - px0 : PX, cy = nby - py0 < PY ? nby - py0 : PY;
        members = static_cast<unsigned>(cx * cy);
        common = static_cast<unsigned>(n_tiles / a.n_splits);
        const uint32_t w = blockIdx.x;
        arrive = a.arrive + (((w >> 3) >> 5) * 8 + (w & 7));
    }
    for (int64_t tile = split; tile < n_tiles; tile += a.n_splits) {
        const int64_t v0 = tile * BV;
        if (arrive && epoch < common) {
            if (epoch % a.align_every == 0) patch_cross(arrive, members * (epoch / a.align_every + 1), a.align_spins);
            ++epoch;
        }
        f32x16 acc[NI][NJ];
        zero_acc<Core>(acc);
        Core::tile(a.op, v0, tok0, acc, lds);
        int t2 = threadIdx.x;
        // (the accumulators are read below by instructions the compiler does not look into: the wait a matrix
        // instruction's result needs before another unit reads it is spelled out)
        asm volatile("s_nop 15\n s_nop 7" : "+v"(t2));
        const int lane2 = t2 & 63, wm2 = t2 >> 7, wn2 = (t2 >> 6) & 1;
        const int col = wn2 * (NJ * 32) + (lane2 & 31);  // this lane's token column of tile j is col + j * 32
        // Accumulator element e of tile i is row `off` = i * 32 + 8 * (e / 4) + e % 4 (a compile-time constant)
        // below this lane's first row vb.  Only the last vocabulary tile needs the rows-past-the-end mask.
        const int vb = static_cast<int>(v0) + wm2 * 128 + 4 * (lane2 >> 5);
        const int limit = static_cast<int>(a.op.m) - vb;  // rows with off < limit exist
        // One 32 x 32 block (16 accumulator registers) at a time, so that only those 16 values are live next to
        // the accumulators: running maximum and sum are rescaled per block (one extra exponential per 16).
        auto fold_tile = [&](auto masked_tag) {
            constexpr bool MASKED = decltype(masked_tag)::value;
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int tg = tgt_s[col + j * 32];
                const int toff = tg - vb;  // the target's row as an offset, if it is in this lane at all
                float run_m = run_m_s[j][t2], run_s = run_s_s[j][t2];
#pragma unroll
                for (int i = 0; i < NI; ++i) {
                    __builtin_amdgcn_sched_barrier(0);
                    // The logits count as rounded to bf16 (the matmul output dtype).  Rounding is monotone, so the
                    // maximum is taken over the raw accumulators and rounded once.
                    float x[16];
                    float raw = -INFINITY;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int off = i * 32 + 8 * (e >> 2) + (e & 3);
                        const float r = acc_read(acc[i][j][e]);
                        x[e] = (!MASKED || off < limit) ? r : -INFINITY;
                        raw = fmaxf(raw, x[e]);
                    }
                    if constexpr (SAVE) {
                        // The block leaves as it lies in the accumulators (kept_block): the lane's 16 values are two
                        // 16-byte pieces, and the wave's 64 pieces of one half are 1 KiB contiguous, so each of the
                        // two stores is one full burst, straight from the registers.
                        const int64_t tb = (tok0 + wn2 * (NJ * 32) + j * 32) >> 5, vblk = (v0 + wm2 * (NI * 32) + i * 32) >> 5;
                        if (tb * 32 < a.op.n && vblk < a.n_vb) {
                            unsigned char* out = a.logits + kept_block(tb, vblk, a.n_vb) + lane2 * 16;
#pragma unroll
                            for (int p = 0; p < 2; ++p)
                                *reinterpret_cast<u32x4*>(out + p * 1024) =
                                    u32x4{pack_bf16x2(x[8 * p], x[8 * p + 1]), pack_bf16x2(x[8 * p + 2], x[8 * p + 3]),
                                          pack_bf16x2(x[8 * p + 4], x[8 * p + 5]), pack_bf16x2(x[8 * p + 6], x[8 * p + 7])};
                        }
                    }
                    const float mx = fmaxf(run_m, round_bf16(raw));
                    const float mx2 = mx * kLog2e;
                    // (the subtraction is exact where an FMA against the rounded mx2 would leave a huge residual
                    // while both maxima are still the -1e30 start value)
                    float sx = run_s * fast_exp2((run_m - mx) * kLog2e);
#pragma unroll
                    for (int e = 0; e < 16; ++e) sx += fast_exp2(__builtin_fmaf(round_bf16(x[e]), kLog2e, -mx2));
                    run_m = mx;
                    run_s = sx;
                    if (tg >= 0 && toff >= i * 32 && toff < i * 32 + 32 && (toff & 4) == 0) {  // rare: the target's row is here
                        // (read again from the accumulators, so that the 16 values above need not stay live for this)
                        float xt = 0.f;
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const float r = acc_read(acc[i][j][e]);
                            xt = toff == i * 32 + 8 * (e >> 2) + (e & 3) ? r : xt;
                        }
                        a.xt[tok0 + col + j * 32] = round_bf16(xt);
                    }
                }
                run_m_s[j][t2] = run_m;
                run_s_s[j][t2] = run_s;
            }
        };
        if (v0 + BV <= a.op.m) fold_tile(std::false_type{});
        else fold_tile(std::true_type{});
    }
    float run_m[NJ], run_s[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) { run_m[j] = run_m_s[j][tid]; run_s[j] = run_s_s[j][tid]; }
    // merge the two half-waves (rows 4 apart), then the two waves that share these token columns
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const float om = __shfl_xor(run_m[j], 32, kWave), os = __shfl_xor(run_s[j], 32, kWave);
        const float mn = fmaxf(run_m[j], om);
        run_s[j] = run_s[j] * fast_exp2((run_m[j] - mn) * kLog2e) + os * fast_exp2((om - mn) * kLog2e);
        run_m[j] = mn;
        if (lane < 32) {
            comb_m[wm][wn * (NJ * 32) + j * 32 + lane] = run_m[j];
            comb_s[wm][wn * (NJ * 32) + j * 32 + lane] = run_s[j];
        }
    }
    __syncthreads();
    if (tid < BT) {
        const int64_t t = tok0 + tid;
        if (t < a.op.n) {
            const float m0 = comb_m[0][tid], m1 = comb_m[1][tid];
            const float mn = fmaxf(m0, m1);
            const float sv = comb_s[0][tid] * fast_exp2((m0 - mn) * kLog2e) + comb_s[1][tid] * fast_exp2((m1 - mn) * kLog2e);
            a.part_m[static_cast<int64_t>(split) * a.op.n + t] = mn;
            a.part_s[static_cast<int64_t>(split) * a.op.n + t] = sv;
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

// token tiles per XCD patch of the recomputing gradient kernel (x 4 vocabulary tiles): 1.7 % faster than 4 x 8
constexpr int kGradPatchTokens = 8;

template <class Core>
__global__ __launch_bounds__(GB_THREADS) void lmhead_grad_kernel(LmGradArgs a) {
    constexpr int NI = Core::NI, NJ = Core::NJ, BM = Core::BM, BN = Core::BN;
    __shared__ __attribute__((aligned(1024))) unsigned char lds[Core::LDS_BYTES];
    __shared__ int tgt_local[BM];
    __shared__ float lse_l[BM], g_l[BM];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    if (!resolve_live(a.op)) return;
    int64_t bx, by;
    if (!patch_tile<kGradPatchTokens>(blockIdx.x, (a.op.m + BM - 1) / BM, (a.op.n + BN - 1) / BN, bx, by)) return;
    const int64_t row0 = bx * BM, col0 = by * BN;
    {
        const int64_t grow = row0 + tid;
        int64_t t = -1;
        // rows past the chunk repeat its last row's operand: give them a log-sum-exp that keeps exp(x - lse)
        // finite, and a zero gradient
        float l = 128.f, g = 0.f;
        if (grow < a.op.m) { t = a.targets[grow] - a.vocab_start; l = a.lse[grow]; g = a.grad[grow]; }
        tgt_local[tid] = (t >= 0 && t < a.op.n && g != 0.f) ? static_cast<int>(t) : -1;
        lse_l[tid] = l * kLog2e;
        g_l[tid] = g;
    }
    __syncthreads();
    f32x16 acc[NI][NJ];
    zero_acc<Core>(acc);
    Core::tile(a.op, row0, col0, acc, lds);
    const int64_t m_pad = ((a.op.m + 63) / 64) * 64;
    // gradient of the lane's 4 consecutive tokens (accumulator rows) of tile (i, j), group q, as two bf16 pairs:
    // s01 / s23 the softmax part alone (for G), p01 / p23 with the one-hot term (for G^T)
    auto grad4 = [&](int i, int j, int q, uint32_t& p01, uint32_t& p23, uint32_t& s01, uint32_t& s23) {
        const int64_t c = col0 + wn * (NJ * 32) + j * 32 + (lane & 31);
        const bool col_ok = c < a.op.n;
        float gv[4], sv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int e = q * 4 + u;
            const int rl = wm * 128 + i * 32 + acc_row(e, lane);
            const bool row_ok = row0 + rl < a.op.m;
            gv[u] = sv[u] = 0.f;
            if (row_ok && col_ok && g_l[rl] != 0.f) {
                const float x = round_bf16(acc[i][j][e]);
                const float p = fast_exp2(__builtin_fmaf(x, kLog2e, -lse_l[rl]));
                sv[u] = -p * g_l[rl];
                gv[u] = tgt_local[rl] == c ? g_l[rl] + round_bf16(sv[u]) : sv[u];
            }
        }
        p01 = pack_bf16x2(gv[0], gv[1]);
        p23 = pack_bf16x2(gv[2], gv[3]);
        s01 = pack_bf16x2(sv[0], sv[1]);
        s23 = pack_bf16x2(sv[2], sv[3]);
    };
    // The softmax part of the whole tile's gradients as bf16 pairs.  A group of 4 accumulator rows is the same for
    // every j, so its per-token values are read from LDS once; columns past the vocabulary become zero by a select.
    auto grad_all = [&](uint32_t (&p01)[NI][NJ][4], uint32_t (&p23)[NI][NJ][4]) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int rl = wm * 128 + i * 32 + acc_row(q * 4, lane);  // first of the 4 consecutive rows
                float lse_r[4], ng_r[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    lse_r[u] = lse_l[rl + u];
                    ng_r[u] = -g_l[rl + u];  // zero for rows past the chunk and for tokens without a gradient
                }
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int c = static_cast<int>(col0) + wn * (NJ * 32) + j * 32 + (lane & 31);
                    float gv[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const float x = round_bf16(acc[i][j][q * 4 + u]);
                        const float p = fast_exp2(__builtin_fmaf(x, kLog2e, -lse_r[u]));
                        gv[u] = c < a.op.n ? p * ng_r[u] : 0.f;
                    }
                    p01[i][j][q] = pack_bf16x2(gv[0], gv[1]);
                    p23[i][j][q] = pack_bf16x2(gv[2], gv[3]);
                }
            }
        }
    };
    if constexpr (Core::LDS_BYTES >= BM * BN * 2) {
        // Both layouts leave through LDS so that every global store is a 16-byte piece of a 512-byte run.
        static_assert(BM == GB_THREADS, "one thread per token row patches the one-hot term");
        // Pass 1, [vocab][token]: a lane's 4 tokens are one 8-byte unit; unit U of row v sits at U ^ (v & 63).
        // Pass 2, [token][vocab]: 2-byte writes; the 16-byte chunk C of row t sits at C ^ ((t >> 2) & 7).
        constexpr int RV = BN / 8;  // 16-byte pieces per token row of the tile
        uint32_t p01[NI][NJ][4], p23[NI][NJ][4];
        grad_all(p01, p23);
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int v = wn * (NJ * 32) + j * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int t0 = wm * 128 + i * 32 + acc_row(q * 4, lane);
                    const int unit = (t0 >> 2) ^ (v & 63);
                    *reinterpret_cast<uint2*>(lds + v * (BM * 2) + unit * 8) = uint2{p01[i][j][q], p23[i][j][q]};
                }
        }
        __syncthreads();
        {   // the one-hot term of G^T: token `tid` adds its g at its target's row, if that row is in this tile
            const int v = tgt_local[tid] - static_cast<int>(col0);
            if (tgt_local[tid] >= 0 && v >= 0 && v < BN) {
                uint16_t* cell = reinterpret_cast<uint16_t*>(lds + v * (BM * 2) + (((tid >> 2) ^ (v & 63)) * 8) + (tid & 3) * 2);
                *cell = static_cast<uint16_t>(f32_to_bf16_bits(g_l[tid] + bf16_bits_to_f32(*cell)));
            }
        }
        __syncthreads();
#pragma unroll 4
        for (int it = 0; it < BN * 32 / GB_THREADS; ++it) {
            const int idx = it * GB_THREADS + tid, v = idx >> 5, m = idx & 31;
            const uint2 lo = *reinterpret_cast<const uint2*>(lds + v * (BM * 2) + (((2 * m) ^ (v & 63)) * 8));
            const uint2 hi = *reinterpret_cast<const uint2*>(lds + v * (BM * 2) + (((2 * m + 1) ^ (v & 63)) * 8));
            const int64_t c = col0 + v, r = row0 + 8 * m;
            if (c < a.op.n && r < a.ldgt) *reinterpret_cast<u32x4*>(a.gt + c * a.ldgt + r) = u32x4{lo.x, lo.y, hi.x, hi.y};
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int v = wn * (NJ * 32) + j * 32 + (lane & 31);
#pragma unroll
            for (int i = 0; i < NI; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int t0 = wm * 128 + i * 32 + acc_row(q * 4, lane);
                    const uint32_t w[2] = {p01[i][j][q], p23[i][j][q]};
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int t = t0 + u;
                        const int chunk = (v >> 3) ^ ((t >> 2) & 7);
                        *reinterpret_cast<uint16_t*>(lds + t * (BN * 2) + chunk * 16 + (v & 7) * 2) =
                            static_cast<uint16_t>(w[u >> 1] >> ((u & 1) * 16));
                    }
                }
        }
        __syncthreads();
#pragma unroll 4
        for (int it = 0; it < BM * RV / GB_THREADS; ++it) {
            const int idx = it * GB_THREADS + tid, t = idx / RV, m = idx % RV;
            const u32x4 x = *reinterpret_cast<const u32x4*>(lds + t * (BN * 2) + ((m ^ ((t >> 2) & 7)) * 16));
            const int64_t r = row0 + t, c = col0 + 8 * m;
            if (r < m_pad && c < a.ldg) *reinterpret_cast<u32x4*>(a.g + r * a.ldg + c) = x;
        }
    } else {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const int64_t c = col0 + wn * (NJ * 32) + j * 32 + (lane & 31);
            const bool col_ok = c < a.op.n;
#pragma unroll
            for (int i = 0; i < NI; ++i) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {  // four groups of four consecutive rows
                    uint32_t p01, p23, s01, s23;
                    grad4(i, j, q, p01, p23, s01, s23);
                    const int64_t r_first = row0 + wm * 128 + i * 32 + acc_row(q * 4, lane);
                    if (c < a.ldg) {
                        uint16_t* gp = a.g + r_first * a.ldg + c;
                        if (r_first + 0 < m_pad) gp[0] = static_cast<uint16_t>(s01);
                        if (r_first + 1 < m_pad) gp[a.ldg] = static_cast<uint16_t>(s01 >> 16);
                        if (r_first + 2 < m_pad) gp[2 * a.ldg] = static_cast<uint16_t>(s23);
                        if (r_first + 3 < m_pad) gp[3 * a.ldg] = static_cast<uint16_t>(s23 >> 16);
                    }
                    if (col_ok && r_first < a.ldgt) {
                        uint2 v;
                        v.x = p01;
                        v.y = p23;
                        *reinterpret_cast<uint2*>(a.gt + c * a.ldgt + r_first) = v;
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// backward from kept logits: the same G and G^T without the product.  One workgroup turns a tile of 128 tokens x
// 128 vocabulary ids: a thread reads 16 bytes of 4 consecutive live tokens (two runs of 4 ids, 8 ids apart: what a
// lane of the forward held; the neighbouring thread holds the runs in between, and the two swap a run each so that
// both end up with 8 consecutive ids), writes its part of G
// straight back (16 bytes of a 256-byte run), and hands the 4 tokens' values of each id to LDS as one 8-byte unit
// of the transposed tile (unit U of row v at U ^ swizzle(v)), from where G^T leaves in 16-byte pieces after the
// one-hot term was added to the tokens' target cells.
// ---------------------------------------------------------------------------------------------
struct LmGradKeptArgs {
    const unsigned char* logits;  // bf16 logits as the forward left them (kept_block)
    int64_t n_vb;
    const int32_t* row_map;   // [rows] token (row of logits) of live row r
    const int32_t* live;      // device count of live tokens
    int64_t live_from, rows;  // this chunk's live rows are [live_from, live_from + rows) clamped to *live
    int64_t vocab;
    const int64_t* targets;   // the live rows' targets, log-sum-exps and upstream gradients
    int64_t vocab_start;
    const float* lse;
    const float* grad;
    uint16_t* g;              // as in LmGradArgs
    int64_t ldg;
    uint16_t* gt;
    int64_t ldgt;
};

constexpr int KT = 128;  // tile side of lmhead_grad_kept_kernel

__global__ __launch_bounds__(256) void lmhead_grad_kept_kernel(LmGradKeptArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[KT * KT * 2];
    __shared__ int tgt_l[KT];
    __shared__ float lse_l[KT], g_l[KT];
    __shared__ int64_t row_l[KT];
    const int tid = threadIdx.x;
    int64_t m = static_cast<int64_t>(a.live[0]) - a.live_from;
    m = m < 0 ? 0 : (m > a.rows ? a.rows : m);
    const int64_t row0 = static_cast<int64_t>(blockIdx.y) * KT, col0 = static_cast<int64_t>(blockIdx.x) * KT;
    if (row0 >= m) return;
    const int64_t m_pad = (m + 63) / 64 * 64;
    if (tid < KT) {
        const int64_t r = row0 + tid;
        int64_t t = -1, src = 0;
        float l = 128.f, g = 0.f;  // rows past the live ones: a finite exponent and a zero gradient
        if (r < m) { t = a.targets[r] - a.vocab_start; l = a.lse[r]; g = a.grad[r]; src = a.row_map[r]; }
        tgt_l[tid] = (t >= 0 && t < a.vocab && g != 0.f) ? static_cast<int>(t) : -1;
        lse_l[tid] = l * kLog2e;
        g_l[tid] = g;
        row_l[tid] = src;
    }
    __syncthreads();
    auto swz = [](int v) { return (v ^ (v >> 5)) & 31; };
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int item = pass * 256 + tid, piece = item & 15, t4 = item >> 4;  // 8 ids x 4 tokens
        const int64_t c = col0 + piece * 8;
        uint32_t w[4][4];  // [token][pair of ids]
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t4 * 4 + u;
            float sv[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) sv[k] = 0.f;
            // (the swap below runs in every lane: whether a token is live is the same for both partners, whether the
            // ids exist is not)
            u32x4 raw = u32x4{0u, 0u, 0u, 0u};
            const bool live = row0 + t < m && g_l[t] != 0.f;
            if (live && (c & ~15) < a.vocab) {
                // piece = 4 * (block of the tile) + 2 * (half p) + h
                const int64_t src = row_l[t];
                raw = *reinterpret_cast<const u32x4*>(a.logits + kept_block(src >> 5, (col0 >> 5) + (piece >> 2), a.n_vb) +
                                                     ((piece >> 1) & 1) * 1024 + ((piece & 1) * 32 + (src & 31)) * 16);
            }
            {
                // this lane (h) holds the ids 16 p + 4 h + {0..3} and + 8 + {0..3}; the lane with the other h sits next
                // to it.  h = 0 keeps its first run and takes the partner's first run, h = 1 takes the partner's
                // second run and keeps its own second: 8 consecutive ids, the ids c .. c + 7 of the tile.
                const bool hi = piece & 1;
                const uint32_t give0 = hi ? raw.x : raw.z, give1 = hi ? raw.y : raw.w;
                const uint32_t got0 = __shfl_xor(give0, 1, kWave), got1 = __shfl_xor(give1, 1, kWave);
                raw = hi ? u32x4{got0, got1, raw.z, raw.w} : u32x4{raw.x, raw.y, got0, got1};
            }
            if (live && c < a.vocab) {
                float x[8];
                Row<NRL_BF16>::decode(raw, x);
                const float ng = -g_l[t], ls = lse_l[t];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    sv[k] = c + k < a.vocab ? fast_exp2(__builtin_fmaf(x[k], kLog2e, -ls)) * ng : 0.f;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) w[u][q] = pack_bf16x2(sv[2 * q], sv[2 * q + 1]);
            if (row0 + t < m_pad && c < a.ldg)
                *reinterpret_cast<u32x4*>(a.g + (row0 + t) * a.ldg + c) = u32x4{w[u][0], w[u][1], w[u][2], w[u][3]};
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int v = piece * 8 + k, q = k >> 1;
            uint2 unit;
            if (k & 1) {
                unit.x = (w[0][q] >> 16) | (w[1][q] & 0xffff0000u);
                unit.y = (w[2][q] >> 16) | (w[3][q] & 0xffff0000u);
            } else {
                unit.x = (w[0][q] & 0xffffu) | (w[1][q] << 16);
                unit.y = (w[2][q] & 0xffffu) | (w[3][q] << 16);
            }
            *reinterpret_cast<uint2*>(lds + v * (KT * 2) + ((t4 ^ swz(v)) * 8)) = unit;
        }
    }
    __syncthreads();
    if (tid < KT) {  // the one-hot term of G^T: token `tid` adds its g at its target's row, if that row is in this tile
        const int v = tgt_l[tid] - static_cast<int>(col0);
        if (tgt_l[tid] >= 0 && v >= 0 && v < KT) {
            uint16_t* cell = reinterpret_cast<uint16_t*>(lds + v * (KT * 2) + (((tid >> 2) ^ swz(v)) * 8) + (tid & 3) * 2);
            *cell = static_cast<uint16_t>(f32_to_bf16_bits(g_l[tid] + bf16_bits_to_f32(*cell)));
        }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < KT * 16 / 256; ++it) {
        const int item = it * 256 + tid, v = item >> 4, mq = item & 15;
        const uint2 lo = *reinterpret_cast<const uint2*>(lds + v * (KT * 2) + (((2 * mq) ^ swz(v)) * 8));
        const uint2 hi = *reinterpret_cast<const uint2*>(lds + v * (KT * 2) + (((2 * mq + 1) ^ swz(v)) * 8));
        const int64_t c = col0 + v, r = row0 + 8 * mq;
        if (c < a.vocab && r < a.ldgt) *reinterpret_cast<u32x4*>(a.gt + c * a.ldgt + r) = u32x4{lo.x, lo.y, hi.x, hi.y};
    }
}

// ---------------------------------------------------------------------------------------------
// plain GEMM with fp32 accumulation: C = A B^T or C += A B^T.  MODE bit 0 (ACCUM): the product is added to what c
// holds; bit 1 (NARROW): the result goes to cb, bf16 with c's row stride, instead of to c.  The two are not
// combined: with the prior values in flight next to the narrowing stores the compiler spills accumulators inside the
// K loop.  A product whose k extent turns out empty on the device still delivers zeros without ACCUM; with ACCUM there
// is nothing to do.
// ---------------------------------------------------------------------------------------------
constexpr int GEMM_ACCUM = 1, GEMM_NARROW = 2;
template <class Core, int MODE>
__global__ __launch_bounds__(GB_THREADS) void gemm_f32_kernel(GemmOperands op, float* c, int64_t ldc, const int32_t* row_map,
                                                              uint16_t* cb) {
    constexpr bool ACCUM = (MODE & GEMM_ACCUM) != 0, NARROW = (MODE & GEMM_NARROW) != 0;
    static_assert(!(ACCUM && NARROW), "accumulate in fp32, narrow in a pass of its own");
    constexpr int NI = Core::NI, NJ = Core::NJ, BM = Core::BM, BN = Core::BN;
    __shared__ __attribute__((aligned(1024))) unsigned char lds[Core::LDS_BYTES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / Core::WAVES_N, wn = wave % Core::WAVES_N;
    const bool runs = resolve_live(op);
    if (!runs) {
        // only an empty k extent leaves anything to write, and only where the output is not simply kept as it is
        if (op.m <= 0 || op.n <= 0 || row_map || ACCUM) return;
    }
    int64_t bx, by;
    if (!patch_tile(blockIdx.x, (op.m + BM - 1) / BM, (op.n + BN - 1) / BN, bx, by)) return;
    const int64_t row0 = bx * BM, col0 = by * BN;
    f32x16 acc[NI][NJ];
    zero_acc<Core>(acc);
    if (runs) Core::tile(op, row0, col0, acc, lds);
    // (the write-back reads the accumulators with instructions the compiler does not look into: the wait a matrix
    // instruction's result needs before another unit reads it is spelled out)
    asm volatile("s_nop 15\n s_nop 7" ::: "memory");
    if (row_map) {
        // rows of the product are scattered: row r of C goes to row row_map[r] of the output (plain store only)
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t r = row0 + wm * (NI * 32) + i * 32 + acc_row(e, lane);
                if (r >= op.m) continue;
                float* out = c + static_cast<int64_t>(row_map[r]) * ldc;
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int64_t col = col0 + wn * (NJ * 32) + j * 32 + (lane & 31);
                    if (col < op.n) out[col] = acc[i][j][e];
                }
            }
        return;
    }
    // an interior tile takes the path without per-element bounds (no divergent branch between the loads)
    const bool interior = row0 + BM <= op.m && col0 + BN <= op.n;
    auto write_back = [&](auto interior_tag) {
        constexpr bool INTERIOR = decltype(interior_tag)::value;
        // Half of the tile's 16 blocks at a time: with an accumulating epilogue all 128 loads of a half go out before
        // the first is used, so a tile pays two memory latencies, not one per block.  The accumulators are read one
        // by one where they are used (plain uses would have the compiler copy them all to vector registers, which
        // are taken by the loaded values).
        constexpr int HI = NI / 2 > 0 ? NI / 2 : 1;
#pragma unroll
        for (int i0 = 0; i0 < NI; i0 += HI) {
            float prior[HI][NJ][16];
            if (ACCUM) {
#pragma unroll
                for (int i = i0; i < i0 + HI; ++i)
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        const int64_t col = col0 + wn * (NJ * 32) + j * 32 + (lane & 31);
                        const float* base = c + (row0 + wm * (NI * 32) + i * 32) * ldc + col;
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int r = acc_row(e, lane);
                            prior[i - i0][j][e] =
                                (INTERIOR || (row0 + wm * (NI * 32) + i * 32 + r < op.m && col < op.n)) ? base[r * ldc] : 0.f;
                        }
                    }
            }
#pragma unroll
            for (int i = i0; i < i0 + HI; ++i)
#pragma unroll
                for (int j = 0; j < NJ; ++j) {
                    const int64_t col = col0 + wn * (NJ * 32) + j * 32 + (lane & 31);
                    // (cb has c's row stride: one set of offsets serves the prior values and the narrowed result)
                    float* base = c + (row0 + wm * (NI * 32) + i * 32) * ldc + col;
                    uint16_t* base_b = cb + (row0 + wm * (NI * 32) + i * 32) * ldc + col;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int r = acc_row(e, lane);
                        const float v = acc_read(acc[i][j][e]);
                        if (INTERIOR || (row0 + wm * (NI * 32) + i * 32 + r < op.m && col < op.n)) {
                            if (NARROW) base_b[r * ldc] = static_cast<uint16_t>(f32_to_bf16_bits(ACCUM ? prior[i - i0][j][e] + v : v));
                            else base[r * ldc] = ACCUM ? prior[i - i0][j][e] + v : v;
                        }
                    }
                }
        }
    };
    if (interior) write_back(std::true_type{});
    else write_back(std::false_type{});
}

// dH[n, :] += g_n * W[target_n, :] in fp32: the one-hot term of dH = G W, kept out of the bf16 product.
// One workgroup per token; tokens without a gradient or with a target outside the shard add nothing.
__global__ __launch_bounds__(256) void lmhead_onehot_dh_kernel(float* dh, int64_t ld_dh, const float* grad, const int64_t* targets,
                                                              int64_t vocab_start, int64_t vocab, const uint16_t* w, int64_t ldw,
                                                              int64_t h) {
    const int64_t n = blockIdx.x;
    const float g = grad[n];
    const int64_t t = targets[n] - vocab_start;
    if (g == 0.f || t < 0 || t >= vocab) return;
    const uint16_t* wr = w + t * ldw;
    float* out = dh + n * ld_dh;
    for (int64_t c = threadIdx.x; c < h; c += 256) out[c] += g * bf16_bits_to_f32(wr[c]);
}

// Order-preserving list of the tokens whose upstream gradient is not zero (one workgroup walks the vector 1024
// entries at a time: a wave's ballot and the waves' running counts give every kept token its slot).  Tokens with a
// zero gradient contribute nothing to dH or dW, so the backward products run on the listed tokens only.
__global__ __launch_bounds__(1024) void live_tokens_kernel(const float* grad, int64_t n, int32_t* idx, int32_t* count) {
    __shared__ int wave_cnt[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int base = 0;
    for (int64_t i0 = 0; i0 < n; i0 += 1024) {
        const int64_t i = i0 + threadIdx.x;
        const bool keep = i < n && grad[i] != 0.0f;
        const unsigned long long ballot = __ballot(keep);
        if (lane == 0) wave_cnt[wave] = __popcll(ballot);
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            before += w < wave ? wave_cnt[w] : 0;
            total += wave_cnt[w];
        }
        if (keep) idx[base + before + __popcll(ballot & ((1ull << lane) - 1ull))] = static_cast<int32_t>(i);
        base += total;
        __syncthreads();
    }
    if (threadIdx.x == 0) *count = base;
}

// Row i of the compact operands is token idx[i] for i < count[0]; rows from count[0] on are zero (they pad the
// last K slab of the dW product, where anything but zero would be multiplied into the result).
__global__ __launch_bounds__(256) void gather_live_kernel(const uint16_t* hidden, int64_t ldh, int64_t h, const int64_t* targets,
                                                         const float* lse, const float* grad, const int32_t* idx,
                                                         const int32_t* count, int64_t n, uint16_t* hidden_c, int64_t* targets_c,
                                                         float* lse_c, float* grad_c) {
    const int64_t i = blockIdx.x;
    const bool live = i < count[0];
    const int64_t src = live ? idx[i] : 0;
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const u32x4* in = reinterpret_cast<const u32x4*>(hidden + src * ldh);
    u32x4* out = reinterpret_cast<u32x4*>(hidden_c + i * h);
    for (int64_t v = threadIdx.x; v < h / 8; v += 256) out[v] = live ? in[v] : zero;
    if (threadIdx.x == 0) {
        targets_c[i] = live ? targets[src] : 0;
        lse_c[i] = live ? lse[src] : 0.f;
        grad_c[i] = live ? grad[src] : 0.f;
    }
}

// B[n, k] = src[k, n] in core C's fragment-major layout (k extent ldk, a multiple of 64): k < rows and n < cols are
// copied, everything else up to pad_k and up to the launch's n tiles is zero.  One workgroup per 64 x 64 tile.
__global__ __launch_bounds__(256) void transpose_to_frag_kernel(const uint16_t* src, int64_t rows, int64_t cols, int64_t lds_,
                                                                uint16_t* dst, int64_t ldk, int64_t pad_k) {
    __shared__ uint16_t tile[64][66];
    const int64_t k0 = static_cast<int64_t>(blockIdx.y) * 64, n0 = static_cast<int64_t>(blockIdx.x) * 64;
    if (k0 >= pad_k) return;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int kk = ty; kk < 64; kk += 4) {
        const int64_t r = k0 + kk, c = n0 + tx;
        tile[kk][tx] = (r < rows && c < cols) ? src[r * lds_ + c] : static_cast<uint16_t>(0);
    }
    __syncthreads();
    const int64_t k16 = ldk / 16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int u = h * 256 + threadIdx.x, blk = u >> 6, lane = u & 63;
        const int ng = blk >> 2, kb = blk & 3;
        const int nl = ng * 32 + (lane & 31), kl = kb * 16 + (lane >> 5) * 8;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = static_cast<uint32_t>(tile[kl + 2 * e][nl]) | (static_cast<uint32_t>(tile[kl + 2 * e + 1][nl]) << 16);
        uint16_t* out = dst + (((n0 / 32 + ng) * k16 + (k0 / 16 + kb)) * 64 + lane) * 8;
        *reinterpret_cast<u32x4*>(out) = u32x4{w[0], w[1], w[2], w[3]};
    }
}

__global__ void f32_to_bf16_kernel(const float* src, uint16_t* dst, int64_t n) {
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<int64_t>(gridDim.x) * blockDim.x)
        dst[i] = static_cast<uint16_t>(f32_to_bf16_bits(src[i]));
}

// one workgroup per row of a [rows, width] fp32 matrix with row stride ld
__global__ __launch_bounds__(256) void fill_zero_rows_kernel(float* p, int64_t ld, int64_t width) {
    float* row = p + static_cast<int64_t>(blockIdx.x) * ld;
    for (int64_t c = threadIdx.x; c < width; c += 256) row[c] = 0.f;
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

// Vocabulary splits of the forward: enough workgroups for every compute unit, in multiples of the
// 8-wide patch side, never more than there are vocabulary tiles.
template <class Core> static int fwd_splits(int64_t n, int64_t v) {
    const int64_t row_blocks = (n + Core::BN - 1) / Core::BN, tiles = (v + Core::BM - 1) / Core::BM;  // token blocks, vocabulary tiles
    int64_t s = (256 + row_blocks - 1) / row_blocks;
    s = (s + 7) / 8 * 8;
    if (s > 64) s = 64;
    if (s > tiles) s = tiles;
    return static_cast<int>(s < 1 ? 1 : s);
}

// arrival counters of the forward's XCD patches (one per 32 workgroups), behind the partials in the workspace
static int64_t fwd_patches(int64_t n_tokens, int splits) {
    const int64_t a = patch_grid((n_tokens + 255) / 256, splits, 4), b = patch_grid((n_tokens + 255) / 256, splits, 8);
    return (a > b ? a : b) / 32;
}

extern "C" int64_t nrl_lmhead_fwd_workspace_bytes(int64_t n_tokens, int64_t vocab) {
    const int64_t n = n_tokens < 1 ? 1 : n_tokens;
    const int sa = fwd_splits<CoreA>(n, vocab), sb = fwd_splits<CoreB>(n, vocab);
    const int sm = sa > sb ? sa : sb;
    return ((2 * sm + 1) * n + fwd_patches(n, sm)) * static_cast<int64_t>(sizeof(float));
}

// How often a patch of the forward re-aligns (see patch_cross): once, before its first tile, unless the environment
// says otherwise (NRL_LMHEAD_ALIGN = 0: never, N: before every N-th tile; for measurements).  Workgroups of a patch
// start apart -- they take over compute units from the patch before as those finish -- and stay apart; aligned once
// they stay together for the whole walk: 65536 tokens x V 151936 with the logits kept fill 120 GB into L2 instead of
// 133 - 173 GB (floor 113.7 GB).  The time does not move (62.1 -> 62.4 ms; aligning before every tile: 64 - 67 ms, the
// crossings cost more than the fills), so this saves traffic, not time.
static unsigned fwd_align_every() {
    static const unsigned n = [] {
        const char* v = getenv("NRL_LMHEAD_ALIGN");
        const int k = v ? atoi(v) : 0;
        return k < 1 ? (1u << 30) : static_cast<unsigned>(k);
    }();
    return n;
}
// polls before a workgroup walks on alone: kAlignSpins unless NRL_LMHEAD_ALIGN_SPINS says otherwise (0: at once; how
// the give-up path is tested)
static unsigned fwd_align_spins() {
    static const unsigned n = [] {
        const char* v = getenv("NRL_LMHEAD_ALIGN_SPINS");
        const long k = v ? atol(v) : -1;
        return k < 0 ? kAlignSpins : static_cast<unsigned>(k > (1 << 20) ? (1 << 20) : k);
    }();
    return n;
}
static bool fwd_align_enabled() {
    static const bool on = [] {
        const char* v = getenv("NRL_LMHEAD_ALIGN");
        return !(v && v[0] == '0' && v[1] == 0);
    }();
    return on;
}

template <class Core> static void launch_fwd(LmFwdArgs& a, float* ws, hipStream_t s) {
    const int64_t n = a.op.n;
    a.n_splits = fwd_splits<Core>(n, a.op.m);
    a.part_m = ws; a.part_s = ws + static_cast<int64_t>(a.n_splits) * n; a.xt = ws + 2 * static_cast<int64_t>(a.n_splits) * n;
    const dim3 grid((unsigned)patch_grid((n + Core::BN - 1) / Core::BN, a.n_splits, fwd_patch_tokens(a.logits != nullptr)));
    // xt and, right behind it, the patches' arrival counters are cleared together
    a.arrive = fwd_align_enabled() ? reinterpret_cast<unsigned int*>(a.xt + n) : nullptr;
    a.align_every = fwd_align_every();
    a.align_spins = fwd_align_spins();
    fill_zero_u32<<<dim3(256), dim3(256), 0, s>>>(reinterpret_cast<uint32_t*>(a.xt), n + (a.arrive ? grid.x / 32 : 0));
    if (a.logits) lmhead_fwd_kernel<Core, true><<<grid, dim3(GB_THREADS), 0, s>>>(a);
    else lmhead_fwd_kernel<Core, false><<<grid, dim3(GB_THREADS), 0, s>>>(a);
}

template <class Core> static void launch_grad(const LmGradArgs& a, hipStream_t s) {
    lmhead_grad_kernel<Core><<<dim3((unsigned)patch_grid((a.op.m + Core::BM - 1) / Core::BM, (a.op.n + Core::BN - 1) / Core::BN, kGradPatchTokens)),
                               dim3(GB_THREADS), 0, s>>>(a);
}

// C = or += A B^T with B in core C's fragment-major layout (op.ldb: its k extent); op.k a multiple of 64
template <int MODE> static void launch_gemm(const GemmOperands& op, float* c, int64_t ldc, hipStream_t s, const int32_t* row_map = nullptr,
                                            uint16_t* cb = nullptr) {
    gemm_f32_kernel<CoreC, MODE><<<dim3((unsigned)patch_grid((op.m + CoreC::BM - 1) / CoreC::BM, (op.n + CoreC::BN - 1) / CoreC::BN)),
                                   dim3(GB_THREADS), 0, s>>>(op, c, ldc, row_map, cb);
}

extern "C" int64_t nrl_lmhead_kept_logits_bytes(int64_t n_tokens, int64_t vocab) {
    return n_tokens < 0 || vocab < 0 ? 0 : kept_logits_bytes(n_tokens, vocab);
}

extern "C" int nrl_lmhead_logprob_fwd(const void* hidden, int64_t n_tokens, int64_t hidden_size, int64_t ldh,
                                      const void* weight, int64_t vocab, int64_t ldw, const int64_t* targets,
                                      int64_t vocab_start, int64_t vocab_end, float* logprob_out, float* lse_out,
                                      void* logits_out, int64_t logits_bytes, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
    if (int e = check_lmhead(hidden, n_tokens, hidden_size, ldh, weight, vocab, ldw, targets)) return e;
    if (vocab_end - vocab_start != vocab) return fail(NRL_E_INVALID, "vocab range does not span the rows of W");
    if (logits_out && (logits_bytes < kept_logits_bytes(n_tokens, vocab) || (reinterpret_cast<uintptr_t>(logits_out) & 15)))
        return fail(NRL_E_INVALID, "kept logits need a 16-byte aligned buffer of nrl_lmhead_kept_logits_bytes() bytes");
    if (n_tokens == 0) return NRL_OK;
    if (!logprob_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (workspace_bytes < nrl_lmhead_fwd_workspace_bytes(n_tokens, vocab)) return fail(NRL_E_WORKSPACE, "workspace too small");
    float* ws = static_cast<float*>(workspace);
    LmFwdArgs a;
    a.op.a = static_cast<const uint16_t*>(weight); a.op.b = static_cast<const uint16_t*>(hidden);
    a.op.lda = ldw; a.op.ldb = ldh; a.op.m = vocab; a.op.n = n_tokens; a.op.k = hidden_size;
    a.targets = targets; a.vocab_start = vocab_start;
    a.logits = static_cast<unsigned char*>(logits_out); a.n_vb = (vocab + 31) / 32;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((n_tokens + 255) / 256 >= (1ll << 24)) return fail(NRL_E_INVALID, "too many tokens");
    if (hidden_size % CoreB::BK == 0) launch_fwd<CoreB>(a, ws, s);
    else launch_fwd<CoreA>(a, ws, s);
    const int splits = a.n_splits;
    lmhead_fwd_finish_kernel<<<dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, s>>>(
        n_tokens, splits, a.part_m, a.part_s, a.xt, targets, vocab_start, vocab_end, logprob_out, lse_out);
    return check_launch("lmhead_logprob_fwd");
}

// tokens per backward chunk: long enough that the dW product (K = chunk) amortises its fp32 read-modify-write
static constexpr int64_t kBwdChunk = 16384;
static int64_t bwd_chunk(int64_t n) { return n < kBwdChunk ? round_up(n < 1 ? 1 : n, 64) : kBwdChunk; }
// Row stride (elements) of the two operands of the dW product, whose rows hold a chunk's tokens: one 128-byte line
// more than the chunk, because rows a power of two apart (16384 tokens = 32 KiB) fall on the same memory channels
// (measured on the dW product: 1.6 % faster than unpadded; two lines more is 5 % slower, three as good as one).
static int64_t bwd_ld_t(int64_t chunk) { return chunk + 64; }

extern "C" int64_t nrl_lmhead_bwd_workspace_bytes(int64_t n_tokens, int64_t hidden_size, int64_t vocab) {
    const int64_t n = n_tokens < 1 ? 1 : n_tokens;
    const int64_t chunk = bwd_chunk(n_tokens), vp = round_up(vocab, 64), n_pad = round_up(n, chunk);
    int64_t b = 0;
    b += round_up(hidden_size, 256) * vp * 2;        // W^T, fragment-major
    b += chunk * vp * 2;              // G
    b += vocab * bwd_ld_t(chunk) * 2;        // G^T
    b += round_up(hidden_size, 256) * bwd_ld_t(chunk) * 2;  // hidden chunk^T, fragment-major
    b += vocab * hidden_size * 4;     // dW accumulator (fp32)
    b += n_pad * hidden_size * 2;     // hidden rows of the tokens that carry a gradient
    b += n_pad * (8 + 4 + 4 + 4);     // their targets, log-sum-exps, gradients and token indices
    return b + 2048;
}

extern "C" int nrl_lmhead_logprob_bwd(const void* hidden, int64_t n_tokens, int64_t hidden_size, int64_t ldh,
                                      const void* weight, int64_t vocab, int64_t ldw, const int64_t* targets,
                                      int64_t vocab_start, int64_t vocab_end, const float* lse, const float* grad,
                                      const void* logits_kept, int64_t logits_bytes, float* dhidden_out, int64_t ld_dh,
                                      void* dweight_out, int64_t ld_dw, void* workspace, int64_t workspace_bytes,
                                      void* stream) {
    if (int e = check_lmhead(hidden, n_tokens, hidden_size, ldh, weight, vocab, ldw, targets)) return e;
    if (vocab_end - vocab_start != vocab) return fail(NRL_E_INVALID, "vocab range does not span the rows of W");
    if (logits_kept && (logits_bytes < kept_logits_bytes(n_tokens, vocab) || (reinterpret_cast<uintptr_t>(logits_kept) & 15)))
        return fail(NRL_E_INVALID, "kept logits need a 16-byte aligned buffer of nrl_lmhead_kept_logits_bytes() bytes");
    if (!dweight_out || !workspace) return fail(NRL_E_INVALID, "null output or workspace");
    if (n_tokens > 0 && (!lse || !grad || !dhidden_out)) return fail(NRL_E_INVALID, "null argument");
    if (n_tokens >= (1ll << 31)) return fail(NRL_E_INVALID, "too many tokens");
    if (ld_dh < hidden_size) return fail(NRL_E_INVALID, "ld_dh shorter than the hidden size");
    if (workspace_bytes < nrl_lmhead_bwd_workspace_bytes(n_tokens, hidden_size, vocab)) return fail(NRL_E_WORKSPACE, "workspace too small");
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return fail(NRL_E_INVALID, "workspace must be 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t chunk = bwd_chunk(n_tokens), vp = round_up(vocab, 64), h = hidden_size;
    const int64_t n_pad = round_up(n_tokens < 1 ? 1 : n_tokens, chunk);
    char* ws = static_cast<char*>(workspace);
    auto take = [&](int64_t bytes) { char* p = ws; ws += (bytes + 255) / 256 * 256; return p; };
    const int64_t h_pad = round_up(h, 256);
    uint16_t* wt = reinterpret_cast<uint16_t*>(take(h_pad * vp * 2));
    uint16_t* g = reinterpret_cast<uint16_t*>(take(chunk * vp * 2));
    const int64_t ld_t = bwd_ld_t(chunk);
    uint16_t* gt = reinterpret_cast<uint16_t*>(take(vocab * ld_t * 2));
    uint16_t* ht = reinterpret_cast<uint16_t*>(take(h_pad * ld_t * 2));
    float* dw = reinterpret_cast<float*>(take(vocab * h * 4));
    uint16_t* hid_c = reinterpret_cast<uint16_t*>(take(n_pad * h * 2));
    int64_t* tgt_c = reinterpret_cast<int64_t*>(take(n_pad * 8));
    float* lse_c = reinterpret_cast<float*>(take(n_pad * 4));
    float* grad_c = reinterpret_cast<float*>(take(n_pad * 4));
    int32_t* idx = reinterpret_cast<int32_t*>(take(n_pad * 4 + 256));
    int32_t* count = idx + n_pad;
    const uint16_t* hid = static_cast<const uint16_t*>(hidden);
    const uint16_t* w = static_cast<const uint16_t*>(weight);

    // W^T [H, vp] (zero-padded, fragment-major: operand B of the dH product)
    transpose_to_frag_kernel<<<dim3((unsigned)(h_pad / 64), (unsigned)(vp / 64)), dim3(256), 0, s>>>(w, vocab, h, ldw, wt, vp, vp);
    if (n_tokens == 0) {
        // no token: dW is zero (rows of h bf16 = h / 2 words, row stride ld_dw / 2 words: both are multiples of 8)
        for (int64_t r = 0; r < vocab; r += 65535)
            fill_zero_rows_kernel<<<dim3((unsigned)(vocab - r < 65535 ? vocab - r : 65535)), dim3(256), 0, s>>>(
                reinterpret_cast<float*>(static_cast<uint16_t*>(dweight_out) + r * ld_dw), ld_dw / 2, h / 2);
    } else {
        // Tokens with a zero upstream gradient (prompt tokens, masked samples, each sequence's dropped last position)
        // have a zero row in G: the three products run on the other tokens only.  How many those are stays on the
        // device; the launches are sized for all tokens and the workgroups beyond the live ones leave at once.
        live_tokens_kernel<<<dim3(1), dim3(1024), 0, s>>>(grad, n_tokens, idx, count);
        gather_live_kernel<<<dim3((unsigned)n_pad), dim3(256), 0, s>>>(hid, ldh, h, targets, lse, grad, idx, count, n_tokens, hid_c, tgt_c,
                                                                        lse_c, grad_c);
        for (int64_t r = 0; r < n_tokens; r += 65535)  // dH rows of the other tokens are zero
            fill_zero_rows_kernel<<<dim3((unsigned)(n_tokens - r < 65535 ? n_tokens - r : 65535)), dim3(256), 0, s>>>(
                dhidden_out + r * ld_dh, ld_dh, h);
    }

    // dW is summed over the chunks in an fp32 buffer and narrowed once at the end.  The first chunk's product starts
    // the buffer (no zero fill, no read; zeros if the chunk turns out to hold no live token); when there is only one
    // chunk its product is written as bf16 straight to the output.
    const bool single = n_tokens <= chunk && ld_dw == h;
    for (int64_t t0 = 0; t0 < n_tokens; t0 += chunk) {
        const int64_t rows = n_tokens - t0 < chunk ? n_tokens - t0 : chunk;   // upper bound: the live rows of this chunk
        const int64_t rows_pad = round_up(rows, 64);
        // G / G^T for this chunk of live tokens
        LmGradArgs ga;
        ga.op.a = hid_c + t0 * h; ga.op.b = w; ga.op.lda = h; ga.op.ldb = ldw; ga.op.m = rows; ga.op.n = vocab; ga.op.k = h;
        ga.op.live = count; ga.op.live_from = t0; ga.op.live_dim = 1;
        ga.targets = tgt_c + t0; ga.vocab_start = vocab_start; ga.lse = lse_c + t0; ga.grad = grad_c + t0;
        ga.g = g; ga.ldg = vp; ga.gt = gt; ga.ldgt = ld_t;
        if (logits_kept) {
            LmGradKeptArgs ka;
            ka.logits = static_cast<const unsigned char*>(logits_kept); ka.n_vb = (vocab + 31) / 32; ka.row_map = idx + t0; ka.live = count;
            ka.live_from = t0; ka.rows = rows; ka.vocab = vocab; ka.targets = ga.targets; ka.vocab_start = vocab_start;
            ka.lse = ga.lse; ka.grad = ga.grad; ka.g = g; ka.ldg = vp; ka.gt = gt; ka.ldgt = ld_t;
            lmhead_grad_kept_kernel<<<dim3((unsigned)((vp + KT - 1) / KT), (unsigned)((rows + KT - 1) / KT)), dim3(256), 0, s>>>(ka);
        } else if (h % CoreB::BK == 0) launch_grad<CoreB>(ga, s);
        else launch_grad<CoreA>(ga, s);
        // dH[token of row r] = G [rows, V] * (W^T [H, V])^T, written to the tokens' own rows
        GemmOperands dh;
        dh.a = g; dh.lda = vp; dh.b = wt; dh.ldb = vp; dh.m = rows; dh.n = h; dh.k = vp;
        dh.live = count; dh.live_from = t0; dh.live_dim = 1;
        launch_gemm<0>(dh, dhidden_out, ld_dh, s, idx + t0);
        // dW += G^T [V, rows] * (hidden^T [H, rows])^T
        transpose_to_frag_kernel<<<dim3((unsigned)(h_pad / 64), (unsigned)(rows_pad / 64)), dim3(256), 0, s>>>(
            hid_c + t0 * h, rows, h, h, ht, ld_t, rows_pad);
        GemmOperands dwo;
        dwo.a = gt; dwo.lda = ld_t; dwo.b = ht; dwo.ldb = ld_t; dwo.m = vocab; dwo.n = h; dwo.k = rows_pad;
        dwo.live = count; dwo.live_from = t0; dwo.live_dim = 2;
        // (the narrowing epilogue writes with the accumulator's row stride)
        if (single) launch_gemm<GEMM_NARROW>(dwo, dw, h, s, nullptr, static_cast<uint16_t*>(dweight_out));
        else if (t0 == 0) launch_gemm<0>(dwo, dw, h, s);
        else launch_gemm<GEMM_ACCUM>(dwo, dw, h, s);
    }
    if (n_tokens > 0 && !single) {
        uint16_t* out = static_cast<uint16_t*>(dweight_out);
        if (ld_dw == h) {
            f32_to_bf16_kernel<<<dim3(2048), dim3(256), 0, s>>>(dw, out, vocab * h);
        } else {
            for (int64_t r = 0; r < vocab; ++r) f32_to_bf16_kernel<<<dim3(4), dim3(256), 0, s>>>(dw + r * h, out + r * ld_dw, h);
        }
    }
    if (n_tokens > 0)  // the one-hot term of dH in fp32, on the tokens' own rows
        for (int64_t r = 0; r < n_tokens; r += 65535)
            lmhead_onehot_dh_kernel<<<dim3((unsigned)(n_tokens - r < 65535 ? n_tokens - r : 65535)), dim3(256), 0, s>>>(
                dhidden_out + r * ld_dh, ld_dh, grad + r, targets + r, vocab_start, vocab, w, ldw, h);
    return check_launch("lmhead_logprob_bwd");
}

// Shared device helpers for the gfx950 kernels: element decoding for fp32 / bf16 / fp16 rows,
// round-to-nearest-even narrowing, wave64 / workgroup reductions and the host-side error slot.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/nrl_hip.h"

namespace nrl {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------------
// host: per-thread error text
// ---------------------------------------------------------------------------------------------
char* error_slot();
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

// ---------------------------------------------------------------------------------------------
// scalar conversions
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }

// fp32 -> bf16 / fp16 bits, round to nearest even (NaN stays a quiet NaN), through the hardware
// converts (v_cvt_pk_bf16_f32, v_cvt_pk_f16_f32): one instruction per pair
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
// (fp16 only: the values are pinned in fp32 registers first.  Otherwise the compiler folds a preceding multiply into
// the conversion as v_fma_mix(a, b, +0): one rounding instead of the two of multiply-then-narrow that PyTorch does,
// and a negative zero product comes out positive.)
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
    asm volatile("" : "+v"(lo), "+v"(hi));
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<__bf16>(f)));
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t lo16) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(lo16)));
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
    asm volatile("" : "+v"(f));  // see pack_f16x2
    return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, static_cast<_Float16>(f)));
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// torch.max / torch.min semantics: NaN propagates
__device__ __forceinline__ float nan_max(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); }
__device__ __forceinline__ float nan_min(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b); }

// ---------------------------------------------------------------------------------------------
// Row element traits.  DT is an nrl_dtype.  A 16-byte vector holds EPV elements.
// TEMP: 0 = no temperature, 1 = round(x / T), 2 = round(x * rcpT); the rounding is to the row's
// own dtype, mirroring an in-place divide of the logits tensor.
// ---------------------------------------------------------------------------------------------
template <int DT> struct Row;

template <> struct Row<NRL_F32> {
    static constexpr int EPV = 4;
    static constexpr int BYTES = 4;
    static constexpr uint32_t NEG_INF_WORD = 0xff800000u;  // -inf in every element of a 32-bit word
    __device__ static __forceinline__ float round_self(float v) { return v; }
    __device__ static __forceinline__ void decode(const u32x4& r, float (&v)[4]) {
        v[0] = __uint_as_float(r.x); v[1] = __uint_as_float(r.y);
        v[2] = __uint_as_float(r.z); v[3] = __uint_as_float(r.w);
    }
    __device__ static __forceinline__ u32x4 encode(const float (&v)[4]) {
        u32x4 r;
        r.x = __float_as_uint(v[0]); r.y = __float_as_uint(v[1]);
        r.z = __float_as_uint(v[2]); r.w = __float_as_uint(v[3]);
        return r;
    }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) { return static_cast<const float*>(p)[i]; }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float v) { static_cast<float*>(p)[i] = v; }
};

template <> struct Row<NRL_BF16> {
    static constexpr int EPV = 8;
    static constexpr int BYTES = 2;
    static constexpr uint32_t NEG_INF_WORD = 0xff80ff80u;
    __device__ static __forceinline__ float round_self(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
    __device__ static __forceinline__ void decode(const u32x4& r, float (&v)[8]) {
        v[0] = __uint_as_float(r.x << 16); v[1] = __uint_as_float(r.x & 0xffff0000u);
        v[2] = __uint_as_float(r.y << 16); v[3] = __uint_as_float(r.y & 0xffff0000u);
        v[4] = __uint_as_float(r.z << 16); v[5] = __uint_as_float(r.z & 0xffff0000u);
        v[6] = __uint_as_float(r.w << 16); v[7] = __uint_as_float(r.w & 0xffff0000u);
    }
    __device__ static __forceinline__ u32x4 encode(const float (&v)[8]) {
        u32x4 r;
        r.x = pack_bf16x2(v[0], v[1]);
        r.y = pack_bf16x2(v[2], v[3]);
        r.z = pack_bf16x2(v[4], v[5]);
        r.w = pack_bf16x2(v[6], v[7]);
        return r;
    }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) {
        return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float v) {
        static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    }
};

template <> struct Row<NRL_F16> {
    static constexpr int EPV = 8;
    static constexpr int BYTES = 2;
    static constexpr uint32_t NEG_INF_WORD = 0xfc00fc00u;
    __device__ static __forceinline__ float round_self(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }
    __device__ static __forceinline__ void decode(const u32x4& r, float (&v)[8]) {
        v[0] = f16_bits_to_f32(r.x & 0xffffu); v[1] = f16_bits_to_f32(r.x >> 16);
        v[2] = f16_bits_to_f32(r.y & 0xffffu); v[3] = f16_bits_to_f32(r.y >> 16);
        v[4] = f16_bits_to_f32(r.z & 0xffffu); v[5] = f16_bits_to_f32(r.z >> 16);
        v[6] = f16_bits_to_f32(r.w & 0xffffu); v[7] = f16_bits_to_f32(r.w >> 16);
    }
    __device__ static __forceinline__ u32x4 encode(const float (&v)[8]) {
        u32x4 r;
        r.x = pack_f16x2(v[0], v[1]);
        r.y = pack_f16x2(v[2], v[3]);
        r.z = pack_f16x2(v[4], v[5]);
        r.w = pack_f16x2(v[6], v[7]);
        return r;
    }
    __device__ static __forceinline__ float load1(const void* p, int64_t i) {
        return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
    }
    __device__ static __forceinline__ void store1(void* p, int64_t i, float v) {
        static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_f16_bits(v));
    }
};

// temperature applied the way an in-place divide of the logits tensor rounds it
template <int DT, int TEMP> __device__ __forceinline__ float scale_logit(float x, float tparam) {
    if constexpr (TEMP == 0) return x;
    else if constexpr (TEMP == 1) return Row<DT>::round_self(__fdiv_rn(x, tparam));
    else return Row<DT>::round_self(x * tparam);
}

// ---------------------------------------------------------------------------------------------
// reductions (wave64)
// ---------------------------------------------------------------------------------------------
template <typename T> __device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v = fminf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Sum over a workgroup of NW waves; every thread receives the total.  `smem` holds NW entries.
// Lanes are combined in a fixed butterfly order and waves in ascending order, so the result
// depends only on the values and the workgroup shape.
template <typename T, int NW> __device__ __forceinline__ T block_sum(T v, T* smem) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    T t = smem[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) t += smem[i];
    return t;
}
template <int NW> __device__ __forceinline__ float block_max(float v, float* smem) {
    v = wave_max(v);
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float t = smem[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) t = fmaxf(t, smem[i]);
    return t;
}
template <int NW> __device__ __forceinline__ float block_min(float v, float* smem) {
    v = wave_min(v);
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) smem[w] = v;
    __syncthreads();
    float t = smem[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) t = fminf(t, smem[i]);
    return t;
}

// Running (maximum, sum of exp(x - maximum)) pair of an online log-sum-exp.
struct Lse {
    float m;  // running maximum
    float s;  // sum of exp(x - m)
};

__device__ __forceinline__ Lse lse_merge(Lse a, Lse b) {
    const float m = fmaxf(a.m, b.m);
    Lse r;
    r.m = m;
    r.s = a.s * fast_exp2((a.m - m) * kLog2e) + b.s * fast_exp2((b.m - m) * kLog2e);
    return r;
}

template <int N> __device__ __forceinline__ void lse_push(Lse& acc, const float (&v)[N]) {
    float vm = v[0];
#pragma unroll
    for (int k = 1; k < N; ++k) vm = fmaxf(vm, v[k]);
    const float mn = fmaxf(acc.m, vm);
    const float mn2 = fmaxf(mn, -1e30f) * kLog2e;  // stays finite while no finite element has been seen
    float part = 0.f;
#pragma unroll
    for (int k = 0; k < N; ++k) part += fast_exp2(__builtin_fmaf(v[k], kLog2e, -mn2));
    acc.s = acc.s * fast_exp2((acc.m - mn) * kLog2e) + part;
    acc.m = mn;
}

__device__ __forceinline__ void lse_push1(Lse& acc, float x) {
    const float mn = fmaxf(acc.m, x);
    acc.s = acc.s * fast_exp2((acc.m - mn) * kLog2e) + fast_exp2((x - mn) * kLog2e);
    acc.m = mn;
}

// merge over the wave, then over the workgroup's NW waves; every thread returns the total
template <int NW> __device__ __forceinline__ Lse block_lse(Lse acc, Lse* smem) {
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
        Lse o;
        o.m = __shfl_xor(acc.m, off, kWave);
        o.s = __shfl_xor(acc.s, off, kWave);
        acc = lse_merge(acc, o);
    }
    const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
    __syncthreads();
    if (lane == 0) smem[w] = acc;
    __syncthreads();
    Lse tot = smem[0];
#pragma unroll
    for (int i = 1; i < NW; ++i) tot = lse_merge(tot, smem[i]);
    return tot;
}

// ---------------------------------------------------------------------------------------------
// d logprob / d logits of one row, times the incoming gradient g: g * (onehot - softmax), narrowed
// once to the row dtype; with a fused temperature the chain rule through the in-place divide rounds
// a second time, as autograd does.  RowGrad carries the per-row constants.
// ---------------------------------------------------------------------------------------------
struct RowGrad {
    float lse2;  // log-sum-exp of the row in base-2 units
    float g, ng;
    float tparam;
    __device__ __forceinline__ RowGrad(float lse, float g_, float tparam_) : lse2(lse * kLog2e), g(g_), ng(-g_), tparam(tparam_) {}
};

template <int DT, int TEMP> __device__ __forceinline__ float grad_finish(float d, float tparam) {
    if constexpr (TEMP == 1) d = __fdiv_rn(Row<DT>::round_self(d), tparam);
    if constexpr (TEMP == 2) d = Row<DT>::round_self(d) * tparam;
    return d;
}

template <int DT, int TEMP> __device__ __forceinline__ float grad_elem(float x, bool is_target, const RowGrad& rg) {
    const float p = fast_exp2(__builtin_fmaf(scale_logit<DT, TEMP>(x, rg.tparam), kLog2e, -rg.lse2));
    return grad_finish<DT, TEMP>(is_target ? (1.f - p) * rg.g : p * rg.ng, rg.tparam);
}

// one 16-byte vector; tsub is the target's place in it, or -1
template <int DT, int TEMP> __device__ __forceinline__ u32x4 grad_vec(const u32x4& raw, int tsub, const RowGrad& rg) {
    constexpr int EPV = Row<DT>::EPV;
    float d[EPV];
    Row<DT>::decode(raw, d);
#pragma unroll
    for (int k = 0; k < EPV; ++k) {
        const float p = fast_exp2(__builtin_fmaf(scale_logit<DT, TEMP>(d[k], rg.tparam), kLog2e, -rg.lse2));
        d[k] = grad_finish<DT, TEMP>(p * rg.ng, rg.tparam);
    }
    if (tsub >= 0) {  // at most one lane of one vector per row
        float t[EPV];
        Row<DT>::decode(raw, t);
#pragma unroll
        for (int k = 0; k < EPV; ++k)
            if (k == tsub) d[k] = grad_elem<DT, TEMP>(t[k], true, rg);
    }
    return Row<DT>::encode(d);
}

// sequence index of packed position p, or -1 if p lies outside every sequence
__device__ __forceinline__ int64_t find_seq(const int32_t* cu, int64_t n_seq, int64_t p) {
    if (n_seq <= 0 || p < cu[0] || p >= cu[n_seq]) return -1;
    int64_t lo = 0, hi = n_seq;  // invariant: cu[lo] <= p < cu[hi]
    while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (cu[mid] <= p) lo = mid; else hi = mid;
    }
    return lo;
}

}  // namespace nrl

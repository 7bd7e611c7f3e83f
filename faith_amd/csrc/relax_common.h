// Device-side pieces shared by the HBM-bound kernels (relaxations, elementwise products):
// q-norm accumulation and 16-byte / 4-byte vector access.
#pragma once
#include "common.h"

namespace {

constexpr int WAVE = 64;
constexpr float TINY = 1e-12f;   // Bounds.py:27

// ------------------------------------------------------------------ q-norm pieces
// Q is FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF or Q_GENERAL (any other dual exponent q, 1 < q < inf,
// carried at run time in `qv`): sum of |v|^q as exp2(q log2|v|) -- two quarter-rate instructions per
// value, still far below what an HBM-bound pass has to spare -- and the 1/q power at the end.
constexpr int Q_GENERAL = 3;
template <int Q>
__device__ __forceinline__ float nacc(float acc, float v, float qv) {
    // one fused instruction: a separate square would be hoisted out of the loop over the perturbed
    // words and held for every value a thread keeps (64 more registers)
    if (Q == FAITH_Q_2) return __builtin_fmaf(v, v, acc);
    if (Q == FAITH_Q_1) return acc + fabsf(v);
    if (Q == Q_GENERAL) return acc + __builtin_amdgcn_exp2f(qv * __builtin_amdgcn_logf(fabsf(v)));   // |0|^q = exp2(-inf) = 0
    // max(acc, |v|) on the bit patterns (non-negative floats order like unsigned integers): fmaxf, and
    // a median-of-three with +inf which the compiler turns back into fmaxf, both come with a
    // canonicalising v_max per value -- 184 more instructions per thread of the register-resident kernels
    return __uint_as_float(max(__float_as_uint(acc), __float_as_uint(v) & 0x7fffffffu));
}
template <int Q>
__device__ __forceinline__ float ncomb(float a, float b) {
    if (Q == FAITH_Q_INF) return __uint_as_float(max(__float_as_uint(a), __float_as_uint(b)));   // both >= 0
    return a + b;
}
template <int Q>
__device__ __forceinline__ float nfin(float a, float qv) {
    if (Q == Q_GENERAL) return a > 0.f ? exp2f(log2f(a) / qv) : 0.f;
    return Q == FAITH_Q_2 ? sqrtf(a) : a;
}

// ------------------------------------------------------------------ cross-lane exchange
// The value another lane of the same row of 16 lanes holds; CTRL is the permutation (a DPP control word).  The
// vector ALU applies it to its own operand: no trip through the LDS crossbar, which every ds_bpermute of a CU shares.
template <int CTRL>
__device__ __forceinline__ float lane_permute(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, false));
}
// What lane ^ M holds.  M = 1, 2 (permutations of four lanes) and 8 (a row of 16 rotated by 8) are lane
// permutations; 4, 16 and 32 go through the crossbar.
template <int M>
__device__ __forceinline__ float lane_xor(float x) {
    if constexpr (M == 1) return lane_permute<0xB1>(x);
    else if constexpr (M == 2) return lane_permute<0x4E>(x);
    else if constexpr (M == 8) return lane_permute<0x128>(x);
    else return __shfl_xor(x, M, WAVE);
}
// Butterfly over the lanes that are M, 2 M, ... 32 apart (the lanes of a wavefront that hold the same columns when
// FIRST threads cover a row), for 2 N partial norms.
template <int Q, int FIRST, int N>
__device__ __forceinline__ void combine_from(float (&a)[N], float (&b)[N]) {
#define FAITH_STEP(M)                                          \
    if constexpr (FIRST <= M) {                                \
        _Pragma("unroll") for (int i = 0; i < N; ++i) {        \
            a[i] = ncomb<Q>(a[i], lane_xor<M>(a[i]));          \
            b[i] = ncomb<Q>(b[i], lane_xor<M>(b[i]));          \
        }                                                      \
    }
    FAITH_STEP(1) FAITH_STEP(2) FAITH_STEP(4) FAITH_STEP(8) FAITH_STEP(16) FAITH_STEP(32)
#undef FAITH_STEP
}

// ------------------------------------------------------------------ vector access
// Stores are non-temporal: lw' / uw' are written once and not read again by this kernel, and
// keeping them out of the cache's way measured 11 % faster at configuration 1 (loads are left
// temporal: marking them non-temporal measured 15 % slower).
typedef float v4f __attribute__((ext_vector_type(4)));
template <int VEC>
struct Vec;
template <>
struct Vec<4> {
    float4 v;
    __device__ __forceinline__ void load(const float *p) { v = *reinterpret_cast<const float4 *>(p); }
    __device__ __forceinline__ void load_nt(const float *p) {
        const v4f t = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
        v = make_float4(t[0], t[1], t[2], t[3]);
    }
    __device__ __forceinline__ void store(float *p) const {
        const v4f t = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(p));
    }
    // through the L2 as an ordinary store: for rows that do not start on 64-byte boundaries, where neighbouring tiles
    // write parts of the same 64 bytes and the cache puts them together before they go to memory
    __device__ __forceinline__ void store_cached(float *p) const { *reinterpret_cast<float4 *>(p) = v; }
    __device__ __forceinline__ void zero() { v = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ float get(int i) const { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }
    __device__ __forceinline__ void set(int i, float f) {
        if (i == 0) v.x = f;
        else if (i == 1) v.y = f;
        else if (i == 2) v.z = f;
        else v.w = f;
    }
};
template <>
struct Vec<1> {
    float v;
    __device__ __forceinline__ void load(const float *p) { v = *p; }
    __device__ __forceinline__ void store(float *p) const { __builtin_nontemporal_store(v, p); }
    __device__ __forceinline__ void store_cached(float *p) const { *p = v; }
    __device__ __forceinline__ void zero() { v = 0.f; }
    __device__ __forceinline__ float get(int) const { return v; }
    __device__ __forceinline__ void set(int, float f) { v = f; }
};

}  // namespace

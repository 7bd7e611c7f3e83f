// Device-side pieces shared by the HBM-bound kernels (relaxations, elementwise products):
// q-norm accumulation and 16-byte / 4-byte vector access.
#pragma once
#include "common.h"

namespace {

constexpr int WAVE = 64;
constexpr float TINY = 1e-12f;   // Bounds.py:27

// ------------------------------------------------------------------ q-norm pieces
template <int Q>
__device__ __forceinline__ float nacc(float acc, float v) {
    if (Q == FAITH_Q_2) return acc + v * v;
    if (Q == FAITH_Q_1) return acc + fabsf(v);
    return fmaxf(acc, fabsf(v));
}
template <int Q>
__device__ __forceinline__ float ncomb(float a, float b) {
    return Q == FAITH_Q_INF ? fmaxf(a, b) : a + b;
}
template <int Q>
__device__ __forceinline__ float nfin(float a) {
    return Q == FAITH_Q_2 ? sqrtf(a) : a;
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
    __device__ __forceinline__ void store(float *p) const {
        const v4f t = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(p));
    }
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
    __device__ __forceinline__ void zero() { v = 0.f; }
    __device__ __forceinline__ float get(int) const { return v; }
    __device__ __forceinline__ void set(int, float f) { v = f; }
};

}  // namespace

// The per-neuron lines of the relaxations (slopes and constant terms from a concrete interval), shared by
// the relaxation kernels and the fused softmax.  fp32 operation order follows the reference line by line
// (Transformer_Verification_Code/Verifiers/Bounds.py:348-381 add_linear, :860-1003, :1136-1161): the functions
// here switch the contraction of a multiply and an add into one fused operation off for their own bodies, whatever
// the translation unit that includes them is built with.
#pragma once
#include "relax_common.h"

namespace {

enum Mode { CONCRETIZE = 0, RELU = FAITH_OP_RELU, TANH = FAITH_OP_TANH, EXP = FAITH_OP_EXP, RECIP = FAITH_OP_RECIPROCAL,
            SQR = FAITH_OP_SQR, SQRT = FAITH_OP_SQRT };

// y = k * (v - x0) + y0
struct Line {
    float k, x0, y0;
};

// ------------------------------------------------------------------ the relaxations
// Bounds.py:921-963.  Strict comparisons: l == 0 or u == 0 is a straddling neuron.
__device__ __forceinline__ void relu_lines(float l, float u, Line &lo, Line &up) {
#pragma clang fp contract(off)
    if (u < 0.f) {
        lo = {0.f, 0.f, 0.f};
        up = {0.f, 0.f, 0.f};
    } else if (l > 0.f) {
        lo = {1.f, 0.f, 0.f};
        up = {1.f, 0.f, 0.f};
    } else {
        up = {u / ((u - l) + TINY), l, 0.f};
        lo = {fabsf(u) > fabsf(l) ? 1.f : 0.f, 0.f, 0.f};
    }
}


// exp with the reference's cap (Bounds.py:984-989): the tangent at 12 above 12.  In double.
__device__ __forceinline__ double exp_capped(float x) {
    return x < 12.f ? exp((double)x) : exp(12.0) * ((double)(x - 12.f) + 1.0);
}

// Bounds.add_linear, constant term (Bounds.py:378, :381): a positive slope takes the same-side
// bound, a non-positive one the opposite bound; three separate roundings.
__device__ __forceinline__ float line_bias(const Line &ln, float same, float other) {
#pragma clang fp contract(off)
    const float b = ln.k > 0.f ? same : other;
    return (b - ln.x0) * ln.k + ln.y0;
}

// Slopes and constant terms of every relaxation whose per-neuron work is a handful of operations
// (everything but tanh).  fp32 operation order follows the reference line by line; exp itself is
// taken in double and rounded once.
template <int MODE>
__device__ __forceinline__ void relax_point(float l, float u, float lb, float ub, float &klo, float &kup, float &olb,
                                            float &oub) {
#pragma clang fp contract(off)
    if (MODE == EXP) {                       // Bounds.py:970-1003
        const float m = fminf((l + u) / 2, l + 0.99f);
        klo = (float)exp((double)fminf(m, 12.f));
        olb = klo * ((lb - m) + 1.f);
        const double el = exp_capped(l), eu = exp_capped(u);
        kup = (float)((eu - el) / (double)((u - l) + TINY));
        oub = (ub * kup - kup * l) + (float)el;
    } else if (MODE == RECIP) {              // Bounds.py:1136-1161 (positive intervals)
        const float m = (l + u) / 2;
        klo = -1.f / (m * m);
        olb = ub * klo + 2.f / m;
        kup = -1.f / (l * u);
        oub = (lb * kup - kup * l) + 1.f / l;
    } else {
        Line lo, up;
        if (MODE == RELU) {
            relu_lines(l, u, lo, up);
        } else if (MODE == SQR) {            // Bounds.py:860-890
            up = {u + l, l, l * l};
            if (u < 0.f) {
                const float m = fmaxf((l + u) / 2, 2 * u);
                lo = {2 * m, m, m * m};
            } else if (l > 0.f) {
                const float m = fminf((l + u) / 2, 2 * l);
                lo = {2 * m, m, m * m};
            } else {
                lo = {0.f, 0.f, 0.f};
            }
        } else {                             // SQRT, Bounds.py:892-919 (positive intervals)
            // the chord slope cancels when u - l is small: the difference is taken in double
            lo = {(float)((sqrt((double)u) - sqrt((double)l)) / (double)((u - l) + TINY)), l, sqrtf(l)};
            const float m = (l + u) / 2;
            up = {0.5f / sqrtf(m), m, sqrtf(m)};
        }
        klo = lo.k;
        kup = up.k;
        olb = line_bias(lo, lb, ub);
        oub = line_bias(up, ub, lb);
    }
}

}  // namespace

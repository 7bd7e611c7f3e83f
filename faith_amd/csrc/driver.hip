// The three places where the layer driver touches device memory without computing bounds: the coefficients of
// the input object, the preconditions of reciprocal / sqrt recorded per batch element, and the verdict.
//
// The reference builds them from tensor expressions (VerifierForward._bound_input,
// Transformer_Verification_Code/Verifiers/VerifierForward.py:127-156; the asserts of Bounds.sqrt / Bounds.reciprocal,
// Verifiers/Bounds.py:892, :1147; VerifierForward._bound_classifier :311-314): three to four launches of a
// microsecond or two each, which at the size of one query is as much as a small layer costs.  Here each is one
// launch.
#include "common.h"

namespace {

// w [batch, rows, dim * words, dim].  Word i of batch element b owns the block [dim * i, dim * (i + 1)) x dim of
// ONE row: row i of a compact object, row positions[b, i] of a dense one; that block is scale[b] * identity,
// everything else zero.  One thread writes VEC consecutive floats of a coefficient row.
template <int VEC>
__global__ void __launch_bounds__(256) input_coefficients(float *__restrict__ w, const long long *__restrict__ pos,
                                                          const float *__restrict__ scales, const float scale,
                                                          const int rows, const int words, const int dim,
                                                          const bool compact, const size_t n) {   // n in units of VEC
    const size_t stride = (size_t)gridDim.x * 256;
    const int cols = dim / VEC;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
        const int c = (int)(e % cols) * VEC;
        size_t t = e / cols;
        const int d = (int)(t % ((size_t)dim * words));
        t /= (size_t)dim * words;
        const int r = (int)(t % rows);
        const size_t b = t / rows;
        const int word = d / dim, diag = d % dim;
        const bool here = compact ? r == word : pos[b * words + word] == (long long)r;
        const float s = here ? (scales ? scales[b] : scale) : 0.f;
        if (VEC == 4) {
            float4 v;
            v.x = diag == c ? s : 0.f;
            v.y = diag == c + 1 ? s : 0.f;
            v.z = diag == c + 2 ? s : 0.f;
            v.w = diag == c + 3 ? s : 0.f;
            reinterpret_cast<float4 *>(w)[e] = v;
        } else {
            w[e] = diag == c ? s : 0.f;
        }
    }
}

// flags[b] = 1 if some value of batch element b fails `v > bound` (strict) / `v >= bound`; a NaN fails both.
// Every writer stores the same byte, so workgroups need no order among themselves.
__global__ void __launch_bounds__(256) flag_below(const float *__restrict__ l, unsigned char *__restrict__ flags,
                                                  const size_t per_batch, const float bound, const bool strict) {
    const size_t b = blockIdx.y;
    const float *src = l + b * per_batch;
    bool bad = false;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < per_batch; e += (size_t)gridDim.x * 256) {
        const float v = src[e];
        bad |= strict ? !(v > bound) : !(v >= bound);
    }
    if (__any(bad) && (threadIdx.x & 63) == 0) flags[b] = 1;
}

__global__ void __launch_bounds__(256) verdict(const float *__restrict__ l, const float *__restrict__ u,
                                               const unsigned char *__restrict__ flags, unsigned char *__restrict__ safe,
                                               const int batch, const size_t stride, const int label) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    if (b >= batch) return;
    const bool ok = label == 0 ? l[b * stride] > 0.f : u[b * stride] < 0.f;
    safe[b] = ok && !(flags && flags[b]) ? 1 : 0;
}

}  // namespace

extern "C" int faith_input_coefficients(float *w, const long long *positions, const float *scales, float scale,
                                        int batch_size, int rows, int words, int dim, int compact, void *stream) {
    FAITH_NOT_NULL(w);
    FAITH_ALIGNED4(w);
    FAITH_REQUIRE(scales == nullptr || faith::aligned(scales, 4), FAITH_ERR_ALIGN,
                  "faith_input_coefficients: scales is not 4-byte aligned");
    FAITH_REQUIRE(batch_size > 0 && rows > 0 && words > 0 && dim > 0, FAITH_ERR_SHAPE,
                  "faith_input_coefficients: batch=%d rows=%d words=%d dim=%d must be positive", batch_size, rows, words, dim);
    if (compact) {
        FAITH_REQUIRE(rows == words, FAITH_ERR_SHAPE,
                      "faith_input_coefficients: a compact object has one row per perturbed word (rows=%d, words=%d)", rows, words);
    } else {
        FAITH_NOT_NULL(positions);
        FAITH_REQUIRE(faith::aligned(positions, 8), FAITH_ERR_ALIGN, "faith_input_coefficients: positions is not 8-byte aligned");
    }
    const size_t floats = (size_t)batch_size * rows * words * dim * dim;
    const bool vec = dim % 4 == 0 && faith::aligned(w, 16);
    const size_t n = vec ? floats / 4 : floats;
    const size_t blocks = (n + 255) / 256;
    const dim3 gd((unsigned)(blocks < 65536 ? blocks : 65536)), bd(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec)
        hipLaunchKernelGGL(input_coefficients<4>, gd, bd, 0, st, w, positions, scales, scale, rows, words, dim, compact != 0, n);
    else
        hipLaunchKernelGGL(input_coefficients<1>, gd, bd, 0, st, w, positions, scales, scale, rows, words, dim, compact != 0, n);
    return faith::check_launch("faith_input_coefficients");
}

extern "C" int faith_flag_below(const float *l, unsigned char *flags, int batch_size, long long per_batch, float bound,
                                int strict, void *stream) {
    FAITH_NOT_NULL(l); FAITH_NOT_NULL(flags);
    FAITH_ALIGNED4(l);
    FAITH_REQUIRE(batch_size > 0 && batch_size <= 65535 && per_batch > 0, FAITH_ERR_SHAPE,
                  "faith_flag_below: batch=%d (1 ... 65535) per_batch=%lld must be positive", batch_size, per_batch);
    const long long blocks = (per_batch + 1023) / 1024;          // about four values per thread
    hipLaunchKernelGGL(flag_below, dim3((unsigned)(blocks < 1024 ? blocks : 1024), (unsigned)batch_size), dim3(256), 0,
                       static_cast<hipStream_t>(stream), l, flags, (size_t)per_batch, bound, strict != 0);
    return faith::check_launch("faith_flag_below");
}

extern "C" int faith_verdict(const float *l, const float *u, const unsigned char *flags, unsigned char *safe,
                             int batch_size, long long stride, int label, void *stream) {
    FAITH_NOT_NULL(l); FAITH_NOT_NULL(u); FAITH_NOT_NULL(safe);
    FAITH_ALIGNED4(l); FAITH_ALIGNED4(u);
    FAITH_REQUIRE(batch_size > 0 && stride > 0, FAITH_ERR_SHAPE, "faith_verdict: batch=%d stride=%lld must be positive",
                  batch_size, stride);
    hipLaunchKernelGGL(verdict, dim3((unsigned)((batch_size + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       l, u, flags, safe, batch_size, (size_t)stride, label);
    return faith::check_launch("faith_verdict");
}

// Row-wise linear operators on a whole bound object, one launch each.
//
// The reference builds these from tensor expressions that each read and write all four tensors
// (Bounds.multiply by a float or a tensor, Bounds.add, the row sums of Bounds.softmax and the mean
// subtraction of Bounds.layer_norm: Transformer_Verification_Code/Verifiers/Bounds.py:594-607,
// :653-664, :383-395, :1005-1014, :1111-1131).  Here the coefficient rows (length * dim_in of them)
// and the constant rows (length of them) of an object go through ONE kernel: these operators are
// bound by HBM on large objects and by launches on small ones, and a Transformer layer is a chain
// of dozens of them.
#include "common.h"

namespace {

constexpr int WAVE = 64;

// W * (W > 0) and the rest, as Bounds.py:653-655 forms them (a zero keeps the sign rule of the product)
__device__ __forceinline__ void split(float s, float &sp, float &sn) {
    sp = s > 0.f ? s : 0.f * s;
    sn = s - sp;
}

struct Pair {                   // the lower and the upper tensor of one kind (coefficients or constants)
    const float *lo, *up;       // source
    const float *add_lo, *add_up;   // second object of Bounds.add, or null
    float *out_lo, *out_up;
};

// ------------------------------------------------------------------ scale, add, shift
// out = src * s+ + src' * s-  (+ other object) (+ per-neuron shift on the constant rows only)
template <int VEC>
__global__ void __launch_bounds__(256) affine_kernel(const Pair w, const Pair b, const float *__restrict__ scale,
                                                     const float scalar, const float *__restrict__ shift,
                                                     const size_t n_w, const size_t n_b, const int H) {
    // n_w, n_b, H in units of VEC floats
    const size_t stride = (size_t)gridDim.x * 256;
    const bool scaled = scale != nullptr || scalar != 1.f;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n_w + n_b; e += stride) {
        const bool is_b = e >= n_w;
        const Pair &p = is_b ? b : w;
        const size_t i = is_b ? e - n_w : e;
        const int col = (int)(i % H) * VEC;
        float l[VEC], u[VEC];
        if (VEC == 4) {
            const float4 a = reinterpret_cast<const float4 *>(p.lo)[i], c = reinterpret_cast<const float4 *>(p.up)[i];
            l[0] = a.x; l[1 % VEC] = a.y; l[2 % VEC] = a.z; l[3 % VEC] = a.w;
            u[0] = c.x; u[1 % VEC] = c.y; u[2 % VEC] = c.z; u[3 % VEC] = c.w;
        } else {
            l[0] = p.lo[i];
            u[0] = p.up[i];
        }
        if (scaled) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                float sp, sn;
                split(scale ? scale[col + v] : scalar, sp, sn);
                const float nl = l[v] * sp + u[v] * sn, nu = l[v] * sn + u[v] * sp;
                l[v] = nl;
                u[v] = nu;
            }
        }
        if (p.add_lo) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                l[v] += p.add_lo[i * VEC + v];
                u[v] += p.add_up[i * VEC + v];
            }
        }
        if (is_b && shift) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float t = shift[col + v];
                l[v] += t;
                u[v] += t;
            }
        }
        if (VEC == 4) {
            reinterpret_cast<float4 *>(p.out_lo)[i] = make_float4(l[0], l[1 % VEC], l[2 % VEC], l[3 % VEC]);
            reinterpret_cast<float4 *>(p.out_up)[i] = make_float4(u[0], u[1 % VEC], u[2 % VEC], u[3 % VEC]);
        } else {
            p.out_lo[i] = l[0];
            p.out_up[i] = u[0];
        }
    }
}

// ------------------------------------------------------------------ row sums and row means
__device__ __forceinline__ float wave_sum(float s) {
#pragma unroll
    for (int m = WAVE / 2; m > 0; m >>= 1) s += __shfl_xor(s, m, WAVE);
    return s;
}

// MODE_SUM: out[r, :] = sum_h src[r, h]                      (Bounds.softmax, Bounds.py:1009-1012)
// MODE_MEAN: out[r, :] = (sum_h src[r, h]) / H               (matmul with the H x H matrix of 1 / H, Bounds.py:1116, :1123)
// MODE_NORM: c = src - mean(other side), then c * weight+- (+ bias on the constant rows)
//            (Bounds.layer_norm without the variance, Bounds.py:1111-1131: the mean is
//             matmul(ones / H), multiply(-1.) swaps the sides, multiply(weight) splits by sign)
constexpr int MODE_SUM = 0, MODE_NORM = 1, MODE_MEAN = 2;
constexpr int CACHE = 4;        // row values a lane keeps between the two passes (rows up to 64 * CACHE * VEC)

template <int MODE, int VEC>
__global__ void __launch_bounds__(256) row_kernel(const Pair w, const Pair b, const float *__restrict__ weight,
                                                  const float *__restrict__ bias, const long long rows_w,
                                                  const long long rows_b, const int H) {
    const long long r = (long long)blockIdx.x * 4 + threadIdx.x / WAVE;
    if (r >= rows_w + rows_b) return;
    const bool is_b = r >= rows_w;
    const Pair &p = is_b ? b : w;
    const size_t base = (size_t)(is_b ? r - rows_w : r) * H;
    const int lane = threadIdx.x % WAVE;
    const int n = H / VEC;      // row length in units of VEC

    float cl[CACHE][VEC], cu[CACHE][VEC];
    auto fetch = [&](int i, float (&l)[VEC], float (&u)[VEC]) {
        if (VEC == 4) {
            const float4 a = *reinterpret_cast<const float4 *>(p.lo + base + (size_t)i * 4);
            const float4 c = *reinterpret_cast<const float4 *>(p.up + base + (size_t)i * 4);
            l[0] = a.x; l[1 % VEC] = a.y; l[2 % VEC] = a.z; l[3 % VEC] = a.w;
            u[0] = c.x; u[1 % VEC] = c.y; u[2 % VEC] = c.z; u[3 % VEC] = c.w;
            if (p.add_lo) {     // Bounds.add of a second object before the row operation: one fp32 add, as the separate launch rounds it
                const float4 a2 = *reinterpret_cast<const float4 *>(p.add_lo + base + (size_t)i * 4);
                const float4 c2 = *reinterpret_cast<const float4 *>(p.add_up + base + (size_t)i * 4);
                l[0] += a2.x; l[1 % VEC] += a2.y; l[2 % VEC] += a2.z; l[3 % VEC] += a2.w;
                u[0] += c2.x; u[1 % VEC] += c2.y; u[2 % VEC] += c2.z; u[3 % VEC] += c2.w;
            }
        } else {
            l[0] = p.lo[base + i];
            u[0] = p.up[base + i];
            if (p.add_lo) {
                l[0] += p.add_lo[base + i];
                u[0] += p.add_up[base + i];
            }
        }
    };
    float sl = 0.f, su = 0.f;
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const int i = lane + c * WAVE;
        if (i < n) {
            fetch(i, cl[c], cu[c]);
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                sl += cl[c][v];
                su += cu[c][v];
            }
        }
    }
    for (int i = lane + CACHE * WAVE; i < n; i += WAVE) {
        float l[VEC], u[VEC];
        fetch(i, l, u);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            sl += l[v];
            su += u[v];
        }
    }
    sl = wave_sum(sl);
    su = wave_sum(su);

    const float inv = 1.f / (float)H;
    const float mean_l = sl * inv, mean_u = su * inv;
    auto emit = [&](int i, const float (&l)[VEC], const float (&u)[VEC]) {
        float ol[VEC], ou[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            if (MODE == MODE_SUM) {
                ol[v] = sl;
                ou[v] = su;
            } else if (MODE == MODE_MEAN) {
                ol[v] = mean_l;
                ou[v] = mean_u;
            } else {
                const int col = i * VEC + v;
                const float c_lo = l[v] - mean_u, c_up = u[v] - mean_l;
                if (weight) {
                    float sp, sn;
                    split(weight[col], sp, sn);
                    ol[v] = c_lo * sp + c_up * sn;
                    ou[v] = c_lo * sn + c_up * sp;
                } else {
                    ol[v] = c_lo;
                    ou[v] = c_up;
                }
                if (is_b && bias) {
                    ol[v] += bias[col];
                    ou[v] += bias[col];
                }
            }
        }
        if (VEC == 4) {
            *reinterpret_cast<float4 *>(p.out_lo + base + (size_t)i * 4) = make_float4(ol[0], ol[1 % VEC], ol[2 % VEC], ol[3 % VEC]);
            *reinterpret_cast<float4 *>(p.out_up + base + (size_t)i * 4) = make_float4(ou[0], ou[1 % VEC], ou[2 % VEC], ou[3 % VEC]);
        } else {
            p.out_lo[base + i] = ol[0];
            p.out_up[base + i] = ou[0];
        }
    };
#pragma unroll
    for (int c = 0; c < CACHE; ++c) {
        const int i = lane + c * WAVE;
        if (i < n) emit(i, cl[c], cu[c]);
    }
    for (int i = lane + CACHE * WAVE; i < n; i += WAVE) {
        float l[VEC], u[VEC];
        if (MODE == MODE_NORM) fetch(i, l, u);
        emit(i, l, u);
    }
}

// ------------------------------------------------------------------ interval arithmetic (method "ibp")
// With interval bound propagation the coefficients are zero and an operator maps the concrete
// interval [l, u] of every neuron to the interval of its image (the `if self.ibp` branches of
// Bounds.py:863-866, :896-898, :924-926, :973-975, :1030-1032, :1139-1143).
__global__ void __launch_bounds__(256) interval_unary_kernel(const int op, const float *__restrict__ l,
                                                             const float *__restrict__ u, float *__restrict__ out_l,
                                                             float *__restrict__ out_u, const size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
        const float a = l[e], b = u[e];
        float lo, hi;
        switch (op) {
            case FAITH_OP_RELU: lo = fmaxf(a, 0.f); hi = fmaxf(b, 0.f); break;
            case FAITH_OP_TANH: lo = tanhf(a); hi = tanhf(b); break;
            case FAITH_OP_EXP: lo = expf(a); hi = expf(b); break;
            case FAITH_OP_RECIPROCAL: lo = 1.f / b; hi = 1.f / a; break;
            case FAITH_OP_SQRT: lo = sqrtf(a); hi = sqrtf(b); break;
            default: {   // FAITH_OP_SQR: zero lower bound when the interval straddles zero (l <= 0 <= u)
                const float aa = a * a, bb = b * b;
                lo = (a > 0.f || b < 0.f) ? fminf(aa, bb) : 0.f;
                hi = fmaxf(aa, bb);
            }
        }
        out_l[e] = lo;
        out_u[e] = hi;
    }
}

// interval of a product: the extreme of the four corner products (Bounds.py:667-676)
__global__ void __launch_bounds__(256) interval_product_kernel(const float *__restrict__ xl, const float *__restrict__ xu,
                                                               const float *__restrict__ yl, const float *__restrict__ yu,
                                                               float *__restrict__ zl, float *__restrict__ zu,
                                                               const size_t n) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
        const float p1 = xl[e] * yl[e], p2 = xl[e] * yu[e], p3 = xu[e] * yl[e], p4 = xu[e] * yu[e];
        zl[e] = fminf(fminf(p1, p2), fminf(p3, p4));
        zu[e] = fmaxf(fmaxf(p1, p2), fmaxf(p3, p4));
    }
}

// ------------------------------------------------------------------ rows of a compact object
// An object whose coefficients vanish outside P positions per batch element keeps [B, P, ...] rows and an
// index positions[B, P] (VerifierForward.py:127-156 builds such an input).  Its concrete intervals are the constants
// everywhere except at those positions: two tensors [B, L, H] are read at / rewritten at the P rows.  Data
// movement only; a position outside 0 .. L-1 names no row (reads as zero, replaces nothing).
__global__ void __launch_bounds__(256) rows_gather2(const float *__restrict__ a, const float *__restrict__ b,
                                                    const long long *__restrict__ pos, float *__restrict__ oa,
                                                    float *__restrict__ ob, const int L, const int P, const int H,
                                                    const size_t n) {          // n = B * P * H
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
        const size_t bp = e / H;
        const int h = (int)(e % H);
        const long long l = pos[bp];
        const bool there = l >= 0 && l < L;
        const size_t src = ((bp / P) * L + (there ? l : 0)) * H + h;
        oa[e] = there ? a[src] : 0.f;
        ob[e] = there ? b[src] : 0.f;
    }
}

__global__ void __launch_bounds__(256) rows_put2(const float *__restrict__ a, const float *__restrict__ b,
                                                 const float *__restrict__ ra, const float *__restrict__ rb,
                                                 const long long *__restrict__ pos, float *__restrict__ oa,
                                                 float *__restrict__ ob, const int L, const int P, const int H,
                                                 const size_t n) {             // n = B * L * H
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
        const size_t bl = e / H;
        const int h = (int)(e % H);
        const size_t bb = bl / L;
        const long long l = (long long)(bl % L);
        int slot = -1;
        for (int p = 0; p < P; ++p)
            if (pos[bb * P + p] == l) slot = p;
        const size_t src = (bb * P + (slot >= 0 ? slot : 0)) * H + h;
        oa[e] = slot >= 0 ? ra[src] : a[e];
        ob[e] = slot >= 0 ? rb[src] : b[e];
    }
}

// out [B, L, W] = t [B, P, W] at the rows the positions name, zero elsewhere; VEC floats per thread.
template <int VEC>
__global__ void __launch_bounds__(256) rows_spread(const float *__restrict__ t, const long long *__restrict__ pos,
                                                   float *__restrict__ out, const int L, const int P, const size_t W,
                                                   const size_t n) {          // W, n in units of VEC floats
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t e = (size_t)blockIdx.x * 256 + threadIdx.x; e < n; e += stride) {
        const size_t bl = e / W, w = e % W;
        const size_t bb = bl / L;
        const long long l = (long long)(bl % L);
        int slot = -1;
        for (int p = 0; p < P; ++p)
            if (pos[bb * P + p] == l) slot = p;
        const size_t src = (bb * P + (slot >= 0 ? slot : 0)) * W + w;
        if (VEC == 4) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (slot >= 0) v = reinterpret_cast<const float4 *>(t)[src];
            reinterpret_cast<float4 *>(out)[e] = v;
        } else {
            out[e] = slot >= 0 ? t[src] : 0.f;
        }
    }
}

bool all_aligned16(std::initializer_list<const void *> ptrs) {
    for (const void *p : ptrs)
        if (p != nullptr && !faith::aligned(p, 16)) return false;
    return true;
}

template <int MODE>
int launch_rows(const char *who, const Pair &w, const Pair &b, const float *weight, const float *bias, long long rows_w,
                long long rows_b, int H, void *stream) {
    FAITH_REQUIRE(rows_w >= 0 && rows_b >= 0 && rows_w + rows_b > 0 && H > 0 && (rows_w + rows_b + 3) / 4 <= 0x7fffffffLL,
                  FAITH_ERR_SHAPE, "%s: rows=%lld + %lld, dim_out=%d out of range", who, rows_w, rows_b, H);
    const bool vec4 = H % 4 == 0 && all_aligned16({w.lo, w.up, w.add_lo, w.add_up, w.out_lo, w.out_up, b.lo, b.up, b.add_lo, b.add_up, b.out_lo,
                                                 b.out_up});
    const dim3 grid((unsigned)((rows_w + rows_b + 3) / 4));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec4)
        hipLaunchKernelGGL((row_kernel<MODE, 4>), grid, dim3(256), 0, st, w, b, weight, bias, rows_w, rows_b, H);
    else
        hipLaunchKernelGGL((row_kernel<MODE, 1>), grid, dim3(256), 0, st, w, b, weight, bias, rows_w, rows_b, H);
    return faith::check_launch(who);
}

}  // namespace

#define FAITH_OBJECT_NOT_NULL()                                                                        \
    FAITH_NOT_NULL(src_lb); FAITH_NOT_NULL(src_ub); FAITH_NOT_NULL(src_lw); FAITH_NOT_NULL(src_uw);    \
    FAITH_NOT_NULL(out_lb); FAITH_NOT_NULL(out_ub); FAITH_NOT_NULL(out_lw); FAITH_NOT_NULL(out_uw);    \
    FAITH_ALIGNED4(src_lb); FAITH_ALIGNED4(src_ub); FAITH_ALIGNED4(src_lw); FAITH_ALIGNED4(src_uw);    \
    FAITH_ALIGNED4(out_lb); FAITH_ALIGNED4(out_ub); FAITH_ALIGNED4(out_lw); FAITH_ALIGNED4(out_uw)

extern "C" int faith_affine_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                         const float *src_uw, const float *scale, float scalar, const float *add_lb,
                                         const float *add_ub, const float *add_lw, const float *add_uw,
                                         const float *shift, float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                                         long long rows_w, long long rows_b, int dim_out, void *stream) {
    FAITH_OBJECT_NOT_NULL();
    const bool adding = add_lb || add_ub || add_lw || add_uw;
    FAITH_REQUIRE(!adding || (add_lb && add_ub && add_lw && add_uw), FAITH_ERR_NULL,
                  "faith_affine_verification: the four tensors of the added object must be given together");
    FAITH_REQUIRE(rows_w >= 0 && rows_b >= 0 && rows_w + rows_b > 0 && dim_out > 0, FAITH_ERR_SHAPE,
                  "faith_affine_verification: rows=%lld + %lld, dim_out=%d out of range", rows_w, rows_b, dim_out);
    const Pair w{src_lw, src_uw, add_lw, add_uw, out_lw, out_uw}, b{src_lb, src_ub, add_lb, add_ub, out_lb, out_ub};
    const bool vec4 = dim_out % 4 == 0 &&
                      all_aligned16({src_lb, src_ub, src_lw, src_uw, add_lb, add_ub, add_lw, add_uw, out_lb, out_ub, out_lw,
                                     out_uw});
    const int vec = vec4 ? 4 : 1;
    const size_t n_w = (size_t)rows_w * dim_out / vec, n_b = (size_t)rows_b * dim_out / vec;
    const size_t blocks = (n_w + n_b + 255) / 256;
    const dim3 grid((unsigned)(blocks < 65536 ? blocks : 65536));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec4)
        hipLaunchKernelGGL(affine_kernel<4>, grid, dim3(256), 0, st, w, b, scale, scalar, shift, n_w, n_b, dim_out / 4);
    else
        hipLaunchKernelGGL(affine_kernel<1>, grid, dim3(256), 0, st, w, b, scale, scalar, shift, n_w, n_b, dim_out);
    return faith::check_launch("faith_affine_verification");
}

extern "C" int faith_rowsum_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                         const float *src_uw, float *out_lb, float *out_ub, float *out_lw,
                                         float *out_uw, long long rows_w, long long rows_b, int dim_out, void *stream) {
    FAITH_OBJECT_NOT_NULL();
    const Pair w{src_lw, src_uw, nullptr, nullptr, out_lw, out_uw}, b{src_lb, src_ub, nullptr, nullptr, out_lb, out_ub};
    return launch_rows<MODE_SUM>("faith_rowsum_verification", w, b, nullptr, nullptr, rows_w, rows_b, dim_out, stream);
}

extern "C" int faith_rowmean_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                          const float *src_uw, float *out_lb, float *out_ub, float *out_lw,
                                          float *out_uw, long long rows_w, long long rows_b, int dim_out, void *stream) {
    FAITH_OBJECT_NOT_NULL();
    const Pair w{src_lw, src_uw, nullptr, nullptr, out_lw, out_uw}, b{src_lb, src_ub, nullptr, nullptr, out_lb, out_ub};
    return launch_rows<MODE_MEAN>("faith_rowmean_verification", w, b, nullptr, nullptr, rows_w, rows_b, dim_out, stream);
}

extern "C" int faith_layer_norm_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                             const float *src_uw, const float *add_lb, const float *add_ub,
                                             const float *add_lw, const float *add_uw, const float *weight,
                                             const float *bias, float *out_lb, float *out_ub, float *out_lw,
                                             float *out_uw, long long rows_w, long long rows_b, int dim_out,
                                             void *stream) {
    FAITH_OBJECT_NOT_NULL();
    const bool adding = add_lb || add_ub || add_lw || add_uw;
    FAITH_REQUIRE(!adding || (add_lb && add_ub && add_lw && add_uw), FAITH_ERR_NULL,
                  "faith_layer_norm_verification: the four tensors of the added object must be given together");
    FAITH_ALIGNED4(add_lb); FAITH_ALIGNED4(add_ub); FAITH_ALIGNED4(add_lw); FAITH_ALIGNED4(add_uw);
    const Pair w{src_lw, src_uw, add_lw, add_uw, out_lw, out_uw}, b{src_lb, src_ub, add_lb, add_ub, out_lb, out_ub};
    return launch_rows<MODE_NORM>("faith_layer_norm_verification", w, b, weight, bias, rows_w, rows_b, dim_out, stream);
}

extern "C" int faith_interval_unary(int op, const float *l, const float *u, float *out_lb, float *out_ub, long long n,
                                    void *stream) {
    FAITH_NOT_NULL(l); FAITH_NOT_NULL(u); FAITH_NOT_NULL(out_lb); FAITH_NOT_NULL(out_ub);
    FAITH_REQUIRE(op >= FAITH_OP_RELU && op <= FAITH_OP_SQRT, FAITH_ERR_UNSUPPORTED, "faith_interval_unary: unknown op %d", op);
    FAITH_REQUIRE(n > 0, FAITH_ERR_SHAPE, "faith_interval_unary: n=%lld must be positive", n);
    const long long blocks = (n + 255) / 256;
    hipLaunchKernelGGL(interval_unary_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), op, l, u, out_lb, out_ub, (size_t)n);
    return faith::check_launch("faith_interval_unary");
}

extern "C" int faith_interval_product(const float *x_l, const float *x_u, const float *y_l, const float *y_u,
                                      float *z_lb, float *z_ub, long long n, void *stream) {
    FAITH_NOT_NULL(x_l); FAITH_NOT_NULL(x_u); FAITH_NOT_NULL(y_l); FAITH_NOT_NULL(y_u);
    FAITH_NOT_NULL(z_lb); FAITH_NOT_NULL(z_ub);
    FAITH_REQUIRE(n > 0, FAITH_ERR_SHAPE, "faith_interval_product: n=%lld must be positive", n);
    const long long blocks = (n + 255) / 256;
    hipLaunchKernelGGL(interval_product_kernel, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), x_l, x_u, y_l, y_u, z_lb, z_ub, (size_t)n);
    return faith::check_launch("faith_interval_product");
}

extern "C" int faith_rows_gather(const float *a, const float *b, const long long *positions, float *out_a, float *out_b,
                                 int batch_size, int length, int n_positions, int dim_out, void *stream) {
    FAITH_NOT_NULL(a); FAITH_NOT_NULL(b); FAITH_NOT_NULL(positions); FAITH_NOT_NULL(out_a); FAITH_NOT_NULL(out_b);
    FAITH_ALIGNED4(a); FAITH_ALIGNED4(b); FAITH_ALIGNED4(out_a); FAITH_ALIGNED4(out_b);
    FAITH_REQUIRE(faith::aligned(positions, 8), FAITH_ERR_ALIGN, "faith_rows_gather: positions is not 8-byte aligned");
    FAITH_REQUIRE(batch_size > 0 && length > 0 && n_positions > 0 && dim_out > 0, FAITH_ERR_SHAPE,
                  "faith_rows_gather: batch=%d length=%d positions=%d dim_out=%d must be positive", batch_size, length,
                  n_positions, dim_out);
    const size_t n = (size_t)batch_size * n_positions * dim_out;
    const size_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(rows_gather2, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a, b, positions, out_a, out_b, length, n_positions, dim_out, n);
    return faith::check_launch("faith_rows_gather");
}

extern "C" int faith_rows_put(const float *a, const float *b, const float *rows_a, const float *rows_b,
                              const long long *positions, float *out_a, float *out_b, int batch_size, int length,
                              int n_positions, int dim_out, void *stream) {
    FAITH_NOT_NULL(a); FAITH_NOT_NULL(b); FAITH_NOT_NULL(rows_a); FAITH_NOT_NULL(rows_b); FAITH_NOT_NULL(positions);
    FAITH_NOT_NULL(out_a); FAITH_NOT_NULL(out_b);
    FAITH_ALIGNED4(a); FAITH_ALIGNED4(b); FAITH_ALIGNED4(rows_a); FAITH_ALIGNED4(rows_b); FAITH_ALIGNED4(out_a); FAITH_ALIGNED4(out_b);
    FAITH_REQUIRE(faith::aligned(positions, 8), FAITH_ERR_ALIGN, "faith_rows_put: positions is not 8-byte aligned");
    FAITH_REQUIRE(batch_size > 0 && length > 0 && n_positions > 0 && dim_out > 0, FAITH_ERR_SHAPE,
                  "faith_rows_put: batch=%d length=%d positions=%d dim_out=%d must be positive", batch_size, length,
                  n_positions, dim_out);
    const size_t n = (size_t)batch_size * length * dim_out;
    const size_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(rows_put2, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), a, b, rows_a, rows_b, positions, out_a, out_b, length, n_positions,
                       dim_out, n);
    return faith::check_launch("faith_rows_put");
}

extern "C" int faith_rows_spread(const float *rows, const long long *positions, float *out, int batch_size, int length,
                                 int n_positions, long long row_floats, void *stream) {
    FAITH_NOT_NULL(rows); FAITH_NOT_NULL(positions); FAITH_NOT_NULL(out);
    FAITH_ALIGNED4(rows); FAITH_ALIGNED4(out);
    FAITH_REQUIRE(faith::aligned(positions, 8), FAITH_ERR_ALIGN, "faith_rows_spread: positions is not 8-byte aligned");
    FAITH_REQUIRE(batch_size > 0 && length > 0 && n_positions > 0 && row_floats > 0, FAITH_ERR_SHAPE,
                  "faith_rows_spread: batch=%d length=%d positions=%d row_floats=%lld must be positive", batch_size, length,
                  n_positions, row_floats);
    const bool vec = row_floats % 4 == 0 && faith::aligned(rows, 16) && faith::aligned(out, 16);
    const size_t W = vec ? (size_t)row_floats / 4 : (size_t)row_floats;
    const size_t n = (size_t)batch_size * length * W;
    const size_t blocks = (n + 255) / 256;
    const dim3 gd((unsigned)(blocks < 262144 ? blocks : 262144)), bd(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec)
        hipLaunchKernelGGL(rows_spread<4>, gd, bd, 0, st, rows, positions, out, length, n_positions, W, n);
    else
        hipLaunchKernelGGL(rows_spread<1>, gd, bd, 0, st, rows, positions, out, length, n_positions, W, n);
    return faith::check_launch("faith_rows_spread");
}

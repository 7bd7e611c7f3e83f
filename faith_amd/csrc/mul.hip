// Elementwise operations on bound objects: product of two bounded quantities (McCormick planes),
// per-column scaling, sum of two objects, and the row sum that softmax needs.  All HBM bound.
//
// Arithmetic of the reference's PyTorch methods: Bounds.multiply (Bounds.py:594-664) with
// get_bounds_xy (:666-688), Bounds.add (:383-395), and the sum / repeat of Bounds.softmax
// (:1005-1014).  The reference has no CUDA kernels for these.
//
// Product of two objects x, y of one shape [rows, D_in, H]: with the concrete intervals
// [l_x, u_x], [l_y, u_y] the planes are  a_l = l_y, a_u = u_y, b = l_x  (b on both sides, as the
// reference has it) and
//   z_lw = (a_l > 0 ? x.lw : x.uw) a_l + (b > 0 ? y.lw : y.uw) b
//   z_uw = (a_u > 0 ? x.uw : x.lw) a_u + (b > 0 ? y.uw : y.lw) b
//   z_lb = ((a_l > 0 ? x.lb : x.ub) a_l - a_l b) + (b > 0 ? y.lb : y.ub) b          (z_ub alike)
// The kernel has the shape of the relaxation kernels: a workgroup owns (row, 32 neurons), the
// D_in rows of the tile of ALL FOUR coefficient tensors stay in registers between the two norm
// reductions and the combination, so every input is read once: 24 bytes per coefficient element.
//
// Built with -ffp-contract=off (the reference rounds every product and sum separately).
#include "relax_common.h"

namespace {

struct MulArgs {
    const float *xlb, *xub, *xlw, *xuw;
    const float *ylb, *yub, *ylw, *yuw;
    float *zlb, *zub, *zlw, *zuw;
    int rows, D, H, words;
    float eps;
    float qv = 0.f;     // the dual exponent when it is none of 1, 2, inf
    int remap = 0;      // register-resident kernel: 2 = whole rows of the object dealt to the XCDs (row r to XCD r % 8)
};

template <int Q, int VEC, int TPR, int NTHREADS, int RPT>
__global__ void __launch_bounds__(NTHREADS) mul_natural(const MulArgs a) {
    constexpr int TH = TPR * VEC;
    constexpr int RG = NTHREADS / TPR;
    constexpr int NW = NTHREADS / WAVE;
    static_assert(TH <= WAVE, "one lane per neuron in wavefront 0");
    extern __shared__ float smem[];
    float *part = smem;                          // [words][NW][4][TH]: x.lw, x.uw, y.lw, y.uw partial norms
    float *coef = part + a.words * NW * 4 * TH;  // [3][TH]: a_l, a_u, b

    const int tiles = (a.H + TH - 1) / TH;
    const int r = blockIdx.x / tiles;
    const int col0 = (blockIdx.x % tiles) * TH;
    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid % TPR, rg = tid / TPR;
    const int col = col0 + c * VEC;
    const bool col_ok = col < a.H;
    const size_t base = (size_t)r * a.D * a.H + col;
    const int blk = a.D / a.words;
    constexpr int CHUNK = RG * RPT;
    const int nchunks = (a.D + CHUNK - 1) / CHUNK;
    const float *src[4] = {a.xlw, a.xuw, a.ylw, a.yuw};

    Vec<VEC> d[4][RPT];

    if (nchunks > 1 && lane < TPR)
        for (int w = 0; w < a.words; ++w)
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < VEC; ++v) part[((w * NW + wv) * 4 + t) * TH + c * VEC + v] = 0.f;

    for (int ch = 0; ch < nchunks; ++ch) {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int row = ch * CHUNK + i * RG + rg;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                if (col_ok && row < a.D)
                    d[t][i].load(src[t] + base + (size_t)row * a.H);
                else
                    d[t][i].zero();
            }
        }
        for (int w = 0; w < a.words; ++w) {
            const int lo_row = w * blk, hi_row = lo_row + blk;
            float pn[4][VEC];
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < VEC; ++v) pn[t][v] = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                const int row = ch * CHUNK + i * RG + rg;
                if (row >= lo_row && row < hi_row) {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) pn[t][v] = nacc<Q>(pn[t][v], d[t][i].get(v), a.qv);
                }
            }
#pragma unroll
            for (int m = TPR; m < WAVE; m <<= 1)
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) pn[t][v] = ncomb<Q>(pn[t][v], __shfl_xor(pn[t][v], m, WAVE));
            if (lane < TPR) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        float *sl = &part[((w * NW + wv) * 4 + t) * TH + c * VEC + v];
                        *sl = nchunks > 1 ? ncomb<Q>(*sl, pn[t][v]) : pn[t][v];
                    }
            }
        }
    }
    __syncthreads();

    // one lane per neuron: both concretizations (Bounds.py:611-612), planes, constant terms
    const int column = col0 + lane;
    if (wv == 0 && lane < TH && column < a.H) {
        const size_t bi = (size_t)r * a.H + column;
        const float xlb = a.xlb[bi], xub = a.xub[bi], ylb = a.ylb[bi], yub = a.yub[bi];
        float lx = xlb, ly = ylb, uy = yub;
        for (int w = 0; w < a.words; ++w) {
            float n[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int g = 0; g < NW; ++g)
#pragma unroll
                for (int t = 0; t < 4; ++t) n[t] = ncomb<Q>(n[t], part[((w * NW + g) * 4 + t) * TH + lane]);
            lx += (-a.eps) * nfin<Q>(n[0], a.qv);
            ly += (-a.eps) * nfin<Q>(n[2], a.qv);
            uy += a.eps * nfin<Q>(n[3], a.qv);
        }
        const float al = ly, au = uy, bt = lx;
        coef[lane] = al;
        coef[TH + lane] = au;
        coef[2 * TH + lane] = bt;
        // Bounds.py:631-646: ((b_src - 0) * k + gamma) then + ((b_src - 0) * k + 0)
        const float gl = -al * bt, gu = -au * bt;
        a.zlb[bi] = ((al > 0.f ? xlb : xub) * al + gl) + (bt > 0.f ? ylb : yub) * bt;
        a.zub[bi] = ((au > 0.f ? xub : xlb) * au + gu) + (bt > 0.f ? yub : ylb) * bt;
    }
    __syncthreads();

    if (!col_ok) return;
    float al[VEC], au[VEC], bt[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        al[v] = coef[c * VEC + v];
        au[v] = coef[TH + c * VEC + v];
        bt[v] = coef[2 * TH + c * VEC + v];
    }
    for (int ch = 0; ch < nchunks; ++ch) {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int row = ch * CHUNK + i * RG + rg;
            if (row < a.D) {
                const size_t off = base + (size_t)row * a.H;
                if (nchunks > 1) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) d[t][i].load(src[t] + off);
                }
                Vec<VEC> ol, ou;
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    const float xl = d[0][i].get(v), xu = d[1][i].get(v), yl = d[2][i].get(v), yu = d[3][i].get(v);
                    ol.set(v, (al[v] > 0.f ? xl : xu) * al[v] + (bt[v] > 0.f ? yl : yu) * bt[v]);
                    ou.set(v, (au[v] > 0.f ? xu : xl) * au[v] + (bt[v] > 0.f ? yu : yl) * bt[v]);
                }
                if (VEC == 4 && a.H % 16 != 0) {     // rows that share 64-byte sectors with their neighbours: through the L2 (see Vec::store_cached; [128, 256, 300]: 76 -> 64 us)
                    ol.store_cached(a.zlw + off);
                    ou.store_cached(a.zuw + off);
                } else {
                    ol.store(a.zlw + off);
                    ou.store(a.zuw + off);
                }
            }
        }
    }
}

// The common shape, straight-line: D_in <= RG * RPT (all four coefficient tensors of the tile stay
// in registers), D_in a multiple of RG, H a multiple of the tile width, 16-byte aligned.  Row
// existence is then a scalar branch and there are neither column predicates nor a second pass.
template <int Q, int TPR, int NTHREADS, int RPT>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(Q == Q_GENERAL ? 2 : 4))) mul_resident(const MulArgs a) {
    constexpr int VEC = 4, TH = TPR * VEC, RG = NTHREADS / TPR, NW = NTHREADS / WAVE;
    static_assert(TH <= WAVE, "one lane per neuron in wavefront 0");
    extern __shared__ float smem[];
    float *part = smem;                          // [words][NW][4][TH]: x.lw, x.uw, y.lw, y.uw partial norms
    float *coef = part + a.words * NW * 4 * TH;  // [3][TH]: a_l, a_u, b

    const int tiles = a.H / TH;
    // consecutive workgroups go to the eight XCDs in turn: with whole rows dealt to the XCDs the workgroups of an XCD
    // stream through consecutive tiles instead of touching every row of the object at once
    int bid = blockIdx.x;
    if (a.remap == 2) {
        const int idx = (int)(blockIdx.x / 8), x = (int)(blockIdx.x % 8);
        bid = (idx / tiles * 8 + x) * tiles + idx % tiles;
    }
    const int r = bid / tiles, col0 = (bid % tiles) * TH;
    const int tid = threadIdx.x, lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid % TPR, rg = tid / TPR;
    const size_t base = ((size_t)r * a.D + rg) * a.H + col0 + c * VEC;
    const size_t row_step = (size_t)RG * a.H;
    const float *__restrict__ src[4] = {a.xlw + base, a.xuw + base, a.ylw + base, a.yuw + base};

    Vec<VEC> d[4][RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (i * RG < a.D)
                d[t][i].load(src[t] + i * row_step);
            else
                d[t][i].zero();
        }
    }
    const int blk = a.D / a.words;
    // a perturbed word owns blk consecutive rows: when that is a multiple of RG, whether step i counts for a word is
    // a scalar test per step instead of one per value (a general exponent: half the quarter-rate arithmetic)
    const bool whole_steps = blk % RG == 0;
    const int steps = blk / RG;
    for (int w = 0; w < a.words; ++w) {
        const int lo_row = w * blk, hi_row = lo_row + blk;
        float pn[4][VEC];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < VEC; ++v) pn[t][v] = 0.f;
        if (whole_steps) {
            const int lo_i = w * steps, hi_i = lo_i + steps;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                if (i >= lo_i && i < hi_i) {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) pn[t][v] = nacc<Q>(pn[t][v], d[t][i].get(v), a.qv);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                const int row = i * RG + rg;
                if (row >= lo_row && row < hi_row) {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            // an opaque copy: |x| of every value would otherwise be formed once, outside the loop
                            // over the words, and held (128 more registers)
                            float x = d[t][i].get(v);
                            asm volatile("" : "+v"(x));
                            pn[t][v] = nacc<Q>(pn[t][v], x, a.qv);
                        }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 4; t += 2) combine_from<Q, TPR>(pn[t], pn[t + 1]);
        if (lane < TPR) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < VEC; ++v) part[((w * NW + wv) * 4 + t) * TH + c * VEC + v] = pn[t][v];
        }
    }
    __syncthreads();

    // one lane per neuron: both concretizations (Bounds.py:611-612), planes, constant terms
    if (wv == 0 && lane < TH) {
        const size_t bi = (size_t)r * a.H + col0 + lane;
        const float xlb = a.xlb[bi], xub = a.xub[bi], ylb = a.ylb[bi], yub = a.yub[bi];
        float lx = xlb, ly = ylb, uy = yub;
        for (int w = 0; w < a.words; ++w) {
            float n[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int g = 0; g < NW; ++g)
#pragma unroll
                for (int t = 0; t < 4; ++t) n[t] = ncomb<Q>(n[t], part[((w * NW + g) * 4 + t) * TH + lane]);
            lx += (-a.eps) * nfin<Q>(n[0], a.qv);
            ly += (-a.eps) * nfin<Q>(n[2], a.qv);
            uy += a.eps * nfin<Q>(n[3], a.qv);
        }
        const float al = ly, au = uy, bt = lx;
        coef[lane] = al;
        coef[TH + lane] = au;
        coef[2 * TH + lane] = bt;
        // Bounds.py:631-646: ((b_src - 0) * k + gamma) then + ((b_src - 0) * k + 0)
        const float gl = -al * bt, gu = -au * bt;
        a.zlb[bi] = ((al > 0.f ? xlb : xub) * al + gl) + (bt > 0.f ? ylb : yub) * bt;
        a.zub[bi] = ((au > 0.f ? xub : xlb) * au + gu) + (bt > 0.f ? yub : ylb) * bt;
    }
    __syncthreads();

    float al[VEC], au[VEC], bt[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        al[v] = coef[c * VEC + v];
        au[v] = coef[TH + c * VEC + v];
        bt[v] = coef[2 * TH + c * VEC + v];
    }
    float *__restrict__ q_lw = a.zlw + base, *__restrict__ q_uw = a.zuw + base;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (i * RG < a.D) {
            Vec<VEC> ol, ou;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float xl = d[0][i].get(v), xu = d[1][i].get(v), yl = d[2][i].get(v), yu = d[3][i].get(v);
                ol.set(v, (al[v] > 0.f ? xl : xu) * al[v] + (bt[v] > 0.f ? yl : yu) * bt[v]);
                ou.set(v, (au[v] > 0.f ? xu : xl) * au[v] + (bt[v] > 0.f ? yu : yl) * bt[v]);
            }
            ol.store(q_lw + i * row_step);
            ou.store(q_uw + i * row_step);
        }
    }
}

template <int Q, int TPR, int NTHREADS, int RPT>
void launch_mul_resident(const MulArgs &a, hipStream_t st) {
    constexpr int TH = TPR * 4;
    const size_t smem = ((size_t)a.words * (NTHREADS / WAVE) * 4 * TH + 3 * TH) * sizeof(float);
    faith::reserve_lds(mul_resident<Q, TPR, NTHREADS, RPT>, smem);
    hipLaunchKernelGGL((mul_resident<Q, TPR, NTHREADS, RPT>), dim3((unsigned)(a.rows * (a.H / TH))), dim3(NTHREADS), smem,
                       st, a);
}

template <int Q, int VEC, int TPR, int NTHREADS, int RPT>
void launch_mul(const MulArgs &a, hipStream_t st) {
    constexpr int TH = TPR * VEC;
    const int tiles = (a.H + TH - 1) / TH;
    const size_t smem = ((size_t)a.words * (NTHREADS / WAVE) * 4 * TH + 3 * TH) * sizeof(float);
    faith::reserve_lds(mul_natural<Q, VEC, TPR, NTHREADS, RPT>, smem);
    hipLaunchKernelGGL((mul_natural<Q, VEC, TPR, NTHREADS, RPT>), dim3((unsigned)(a.rows * tiles)), dim3(NTHREADS), smem,
                       st, a);
}

template <int Q>
void dispatch_mul(const MulArgs &a, hipStream_t st) {
    const bool vec4 = a.H % 4 == 0 && faith::aligned(a.xlw, 16) && faith::aligned(a.xuw, 16) &&
                      faith::aligned(a.ylw, 16) && faith::aligned(a.yuw, 16) && faith::aligned(a.zlw, 16) &&
                      faith::aligned(a.zuw, 16);
    const int tv = faith::tune_get(FAITH_TUNE_ACT_VARIANT);
    if (vec4 && a.H % 32 == 0 && a.D % 64 == 0 && a.D <= 256 && tv != 9) {
        // 32-neuron tiles, 512 threads holding 4 rows of each of the four tensors (64 values per thread)
        MulArgs b = a;
        b.remap = (a.rows % 8 == 0 && tv != 8) ? 2 : 0;
        launch_mul_resident<Q, 8, 512, 4>(b, st);
        return;
    }
    if (!vec4)
        launch_mul<Q, 1, 64, 256, 8>(a, st);      // 64 neurons x 32 rows per pass
    else if (a.D <= 128)
        launch_mul<Q, 4, 8, 256, 4>(a, st);       // 32 neurons, D_in <= 128 in registers (64 values per thread)
    else
        launch_mul<Q, 4, 8, 256, 8>(a, st);       // D_in <= 256 in registers (128 values per thread), passes beyond
}

}  // namespace

extern "C" int faith_multiply_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                           const float *y_lb, const float *y_ub, const float *y_lw, const float *y_uw,
                                           float *z_lb, float *z_ub, float *z_lw, float *z_uw, int length, int dim_in,
                                           int dim_out, float epsilon, int q, int words, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw);
    FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_NOT_NULL(z_lb); FAITH_NOT_NULL(z_ub); FAITH_NOT_NULL(z_lw); FAITH_NOT_NULL(z_uw);
    FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_ALIGNED4(z_lw); FAITH_ALIGNED4(z_uw);
    FAITH_REQUIRE(length > 0 && dim_in > 0 && dim_out > 0, FAITH_ERR_SHAPE,
                  "faith_multiply_verification: length=%d dim_in=%d dim_out=%d must be positive", length, dim_in, dim_out);
    FAITH_REQUIRE(words >= 1 && words <= 16 && dim_in % words == 0, FAITH_ERR_SHAPE,
                  "faith_multiply_verification: words=%d must be in 1..16 and divide dim_in=%d", words, dim_in);
    float qv = 0.f;
    if (!faith::dual_exponent(q, &qv)) {
        faith::set_error("faith_multiply_verification: q=%d is neither FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF nor the bits of "
                         "an exponent in (1, inf)", q);
        return FAITH_ERR_UNSUPPORTED;
    }
    MulArgs a{x_lb, x_ub, x_lw, x_uw, y_lb, y_ub, y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, length, dim_in, dim_out, words,
              epsilon};
    hipStream_t st = static_cast<hipStream_t>(stream);
    a.qv = qv;
    if (q == FAITH_Q_1) dispatch_mul<FAITH_Q_1>(a, st);
    else if (q == FAITH_Q_2) dispatch_mul<FAITH_Q_2>(a, st);
    else if (q == FAITH_Q_INF) dispatch_mul<FAITH_Q_INF>(a, st);
    else dispatch_mul<Q_GENERAL>(a, st);
    return faith::check_launch("faith_multiply_verification");
}

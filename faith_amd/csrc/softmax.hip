// Softmax over the last axis of a bound object, as ONE pass over HBM.
//
// The reference composes it from four of its operators
// (Transformer_Verification_Code/Verifiers/Bounds.py:1005-1014):
//     e = x.exp()                      :970-1003   relaxation, needs the concrete interval of x
//     s = sum of e over H, repeated    :1007-1012  every column of s is the same neuron
//     r = s.reciprocal()               :1136-1161  relaxation, needs the concrete interval of s
//     z = e.multiply(r)                :608-651    McCormick planes, need the intervals of e and r
// -- four full-size tensors written and five read per coefficient tensor.  The object a position
// (row r) owns is a [D_in, H] slab of lw and of uw with H the number of key positions: small
// enough to stay in the registers of one workgroup from the load of x to the store of z.  The
// workgroup runs the four operators on what it holds, with the reference's fp32 operation
// order inside each (the same per-neuron code as the separate kernels) and every intermediate
// rounded to fp32 where the reference stores a tensor; s and r are kept as what they are, one
// neuron per row (D_in coefficients per thread column instead of D_in x H).
//
// Layout: TPR = 2^k threads cover one slab row (TPR * VEC >= H columns, lanes along H), RG =
// NTHREADS / TPR rows are in flight, a thread keeps RPT of them.  D_in <= RG * RPT.
//
// Built with -ffp-contract=off (see relax_lines.h).
#include "relax_lines.h"

namespace {

struct SoftmaxArgs {
    const float *lb, *ub, *lw, *uw;
    float *olb, *oub, *olw, *ouw;
    float *sum_l;                   // [rows] concrete lower bound of the sum (the reciprocal's precondition), or null
    int rows, D, H, words;
    float eps, qv;
    float scale;                    // > 0: the object is multiplied by it first (Bounds.multiply with a float)
};

template <int Q, int VEC, int NTHREADS, int RPT>
__global__ void __launch_bounds__(NTHREADS) softmax_kernel(const SoftmaxArgs a, const int tpr_log2) {
    constexpr int NW = NTHREADS / WAVE;
    extern __shared__ float smem[];
    const int TPR = 1 << tpr_log2, TH = TPR * VEC, RG = NTHREADS >> tpr_log2;
    float *part = smem;                              // [words][NW][2][TH] column partial norms (x, then e)
    float *col = part + a.words * NW * 2 * TH;       // [5][TH]: k_lo, k_up of exp; e.lb, e.ub; b = l_e
    float *spart = col + 5 * TH;                     // [words][NW][2] partial norms of the one-neuron objects s, r
    float *scal = spart + a.words * NW * 2;          // [2]: s.lb, s.ub

    const int r = blockIdx.x;
    const int tid = threadIdx.x, lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid & (TPR - 1), rg = tid >> tpr_log2;
    const int col0 = c * VEC;
    const bool col_ok = col0 < a.H;                  // VEC == 4: H % 4 == 0, so the four columns stand or fall together
    const size_t base = ((size_t)r * a.D + rg) * a.H + col0;
    const size_t row_step = (size_t)RG * a.H;
    const int blk = a.D / a.words;

    // ---- x: the slab into registers
    Vec<VEC> dl[RPT], du[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (col_ok && i * RG + rg < a.D) {
            dl[i].load(a.lw + base + i * row_step);
            du[i].load(a.uw + base + i * row_step);
#pragma unroll
            for (int v = 0; v < VEC; ++v) {        // one rounding, as the separate scaling stores it
                dl[i].set(v, dl[i].get(v) * a.scale);
                du[i].set(v, du[i].get(v) * a.scale);
            }
        } else {
            dl[i].zero();
            du[i].zero();
        }
    }

    // column norms of what dl / du hold -> part; the caller synchronises
    auto column_norms = [&]() {
        for (int w = 0; w < a.words; ++w) {
            const int lo_row = w * blk, hi_row = lo_row + blk;
            float pl[VEC], pu[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v) pl[v] = pu[v] = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                const int row = i * RG + rg;
                if (row >= lo_row && row < hi_row) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        pl[v] = nacc<Q>(pl[v], dl[i].get(v), a.qv);
                        pu[v] = nacc<Q>(pu[v], du[i].get(v), a.qv);
                    }
                }
            }
            for (int m = TPR; m < WAVE; m <<= 1) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    pl[v] = ncomb<Q>(pl[v], __shfl_xor(pl[v], m, WAVE));
                    pu[v] = ncomb<Q>(pu[v], __shfl_xor(pu[v], m, WAVE));
                }
            }
            if (lane < TPR) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    part[((w * NW + wv) * 2 + 0) * TH + col0 + v] = pl[v];
                    part[((w * NW + wv) * 2 + 1) * TH + col0 + v] = pu[v];
                }
            }
        }
    };
    // norms over D_in of a one-neuron object whose coefficients sit in sl / su (every thread of a slab row holds
    // the same values: the threads of column group 0 speak for the row) -> spart; the caller synchronises
    float sl[RPT], su[RPT];
    auto neuron_norms = [&]() {
        for (int w = 0; w < a.words; ++w) {
            const int lo_row = w * blk, hi_row = lo_row + blk;
            float pl = 0.f, pu = 0.f;
            if (c == 0) {
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    const int row = i * RG + rg;
                    if (row >= lo_row && row < hi_row) {
                        pl = nacc<Q>(pl, sl[i], a.qv);
                        pu = nacc<Q>(pu, su[i], a.qv);
                    }
                }
            }
#pragma unroll
            for (int m = 1; m < WAVE; m <<= 1) {
                pl = ncomb<Q>(pl, __shfl_xor(pl, m, WAVE));
                pu = ncomb<Q>(pu, __shfl_xor(pu, m, WAVE));
            }
            if (lane == 0) {
                spart[(w * NW + wv) * 2 + 0] = pl;
                spart[(w * NW + wv) * 2 + 1] = pu;
            }
        }
    };
    // [lb - eps * sum of norms, ub + eps * sum of norms] from partial norms (Bounds.py:311-326)
    auto interval = [&](const float *p, int stride, int offset, float lb, float ub, float &l, float &u) {
        l = lb;
        u = ub;
        for (int w = 0; w < a.words; ++w) {
            float nl = 0.f, nu = 0.f;
            for (int g = 0; g < NW; ++g) {
                nl = ncomb<Q>(nl, p[((w * NW + g) * 2 + 0) * stride + offset]);
                nu = ncomb<Q>(nu, p[((w * NW + g) * 2 + 1) * stride + offset]);
            }
            l += (-a.eps) * nfin<Q>(nl, a.qv);
            u += a.eps * nfin<Q>(nu, a.qv);
        }
    };

    // ---- e = exp(x): Bounds.py:970-1003
    column_norms();
    __syncthreads();
    const size_t bi = (size_t)r * a.H + tid;         // thread h < H speaks for column h
    if (tid < a.H) {
        const float xlb = a.lb[bi] * a.scale, xub = a.ub[bi] * a.scale;
        float l, u, klo, kup, elb, eub;
        interval(part, TH, tid, xlb, xub, l, u);
        relax_point<EXP>(l, u, xlb, xub, klo, kup, elb, eub);
        col[tid] = klo;
        col[TH + tid] = kup;
        col[2 * TH + tid] = elb;
        col[3 * TH + tid] = eub;
    }
    __syncthreads();
    if (col_ok) {
        float klo[VEC], kup[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            klo[v] = col[col0 + v];
            kup[v] = col[TH + col0 + v];
        }
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float xl = dl[i].get(v), xu = du[i].get(v);
                dl[i].set(v, (klo[v] > 0.f ? xl : xu) * klo[v]);
                du[i].set(v, (kup[v] > 0.f ? xu : xl) * kup[v]);
            }
        }
    }

    // ---- s = sum of e over H (Bounds.py:1007-1012): coefficients per slab row, constants by wavefront 0
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        float tl = 0.f, tu = 0.f;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            tl += dl[i].get(v);
            tu += du[i].get(v);
        }
        for (int m = 1; m < TPR; m <<= 1) {
            tl += __shfl_xor(tl, m, WAVE);
            tu += __shfl_xor(tu, m, WAVE);
        }
        sl[i] = tl;
        su[i] = tu;
    }
    if (wv == 0) {
        float tl = 0.f, tu = 0.f;
        for (int h = lane; h < a.H; h += WAVE) {
            tl += col[2 * TH + h];
            tu += col[3 * TH + h];
        }
#pragma unroll
        for (int m = 1; m < WAVE; m <<= 1) {
            tl += __shfl_xor(tl, m, WAVE);
            tu += __shfl_xor(tu, m, WAVE);
        }
        if (lane == 0) {
            scal[0] = tl;
            scal[1] = tu;
        }
    }
    neuron_norms();
    __syncthreads();

    // ---- r = 1 / s: Bounds.py:1136-1161, every thread for itself (one neuron)
    float rlb, rub;
    {
        const float slb = scal[0], sub = scal[1];
        float l, u, klo, kup;
        interval(spart, 1, 0, slb, sub, l, u);
        if (tid == 0 && a.sum_l) a.sum_l[r] = l;
        relax_point<RECIP>(l, u, slb, sub, klo, kup, rlb, rub);
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const float xl = sl[i], xu = su[i];
            sl[i] = (klo > 0.f ? xl : xu) * klo;
            su[i] = (kup > 0.f ? xu : xl) * kup;
        }
    }
    __syncthreads();                                 // part and spart are read no more: they take the norms of e and r

    // ---- z = e * r: Bounds.py:608-651 with a_l = l_r, a_u = u_r, b = l_e
    column_norms();
    neuron_norms();
    __syncthreads();
    float al, au;
    interval(spart, 1, 0, rlb, rub, al, au);
    if (tid < a.H) {
        const float elb = col[2 * TH + tid], eub = col[3 * TH + tid];
        float bt, unused;
        interval(part, TH, tid, elb, eub, bt, unused);
        col[4 * TH + tid] = bt;
        const float gl = -al * bt, gu = -au * bt;
        a.olb[bi] = ((al > 0.f ? elb : eub) * al + gl) + (bt > 0.f ? rlb : rub) * bt;
        a.oub[bi] = ((au > 0.f ? eub : elb) * au + gu) + (bt > 0.f ? rub : rlb) * bt;
    }
    __syncthreads();
    if (!col_ok) return;
    float bt[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) bt[v] = col[4 * TH + col0 + v];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (i * RG + rg < a.D) {
            Vec<VEC> ol, ou;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float el = dl[i].get(v), eu = du[i].get(v);
                ol.set(v, (al > 0.f ? el : eu) * al + (bt[v] > 0.f ? sl[i] : su[i]) * bt[v]);
                ou.set(v, (au > 0.f ? eu : el) * au + (bt[v] > 0.f ? su[i] : sl[i]) * bt[v]);
            }
            ol.store(a.olw + base + i * row_step);
            ou.store(a.ouw + base + i * row_step);
        }
    }
}

template <int Q, int VEC, int NTHREADS, int RPT>
bool launch(const SoftmaxArgs &a, int tpr_log2, hipStream_t st) {
    const int TH = (1 << tpr_log2) * VEC, NW = NTHREADS / WAVE;
    const size_t smem = ((size_t)a.words * NW * 2 * TH + 5 * TH + (size_t)a.words * NW * 2 + 2) * sizeof(float);
    // wide slabs with several perturbed words go beyond 64 KB (H = 256, two words: 71 KB); beyond the
    // 160 KB a workgroup can have the caller composes the four operators
    if (!faith::reserve_lds(softmax_kernel<Q, VEC, NTHREADS, RPT>, smem)) return false;
    hipLaunchKernelGGL((softmax_kernel<Q, VEC, NTHREADS, RPT>), dim3((unsigned)a.rows), dim3(NTHREADS), smem, st, a, tpr_log2);
    return true;
}

// The smallest workgroup whose threads hold the slab: RG * RPT >= D_in with RG = NTHREADS / TPR.
template <int Q>
bool dispatch(const SoftmaxArgs &a, bool vec4, hipStream_t st) {
    const int vec = vec4 ? 4 : 1;
    int k = 0;
    while (((1 << k) * vec) < a.H) ++k;
    if ((1 << k) > WAVE) return false;               // a slab row wider than a wavefront covers
    const int tpr = 1 << k;
    if (vec4) {
        if ((256 / tpr) * 8 >= a.D) return launch<Q, 4, 256, 8>(a, k, st);
        if ((1024 / tpr) * 8 >= a.D) return launch<Q, 4, 1024, 8>(a, k, st);
        return false;
    }
    if ((256 / tpr) * 16 >= a.D) return launch<Q, 1, 256, 16>(a, k, st);
    if ((1024 / tpr) * 8 >= a.D) return launch<Q, 1, 1024, 8>(a, k, st);
    if ((1024 / tpr) * 24 >= a.D) return launch<Q, 1, 1024, 24>(a, k, st);
    return false;
}

}  // namespace

extern "C" int faith_softmax_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                          const float *src_uw, float *out_lb, float *out_ub, float *out_lw,
                                          float *out_uw, float *sum_l, float scale, int length, int dim_in,
                                          int dim_out, float epsilon, int q, int words, void *stream) {
    FAITH_NOT_NULL(src_lb); FAITH_NOT_NULL(src_ub); FAITH_NOT_NULL(src_lw); FAITH_NOT_NULL(src_uw);
    FAITH_NOT_NULL(out_lb); FAITH_NOT_NULL(out_ub); FAITH_NOT_NULL(out_lw); FAITH_NOT_NULL(out_uw);
    FAITH_ALIGNED4(src_lb); FAITH_ALIGNED4(src_ub); FAITH_ALIGNED4(src_lw); FAITH_ALIGNED4(src_uw);
    FAITH_ALIGNED4(out_lb); FAITH_ALIGNED4(out_ub); FAITH_ALIGNED4(out_lw); FAITH_ALIGNED4(out_uw);
    FAITH_ALIGNED4(sum_l);
    FAITH_REQUIRE(length > 0 && dim_in > 0 && dim_out > 0, FAITH_ERR_SHAPE,
                  "faith_softmax_verification: length=%d dim_in=%d dim_out=%d must all be positive", length, dim_in,
                  dim_out);
    FAITH_REQUIRE(words >= 1 && words <= 16 && dim_in % words == 0, FAITH_ERR_SHAPE,
                  "faith_softmax_verification: words=%d must be in 1..16 and divide dim_in=%d", words, dim_in);
    FAITH_REQUIRE(scale > 0.f, FAITH_ERR_UNSUPPORTED,
                  "faith_softmax_verification: scale=%g must be positive (a negative factor swaps lower and upper: scale "
                  "the object with faith_affine_verification first)", (double)scale);
    SoftmaxArgs a{src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw, sum_l, length, dim_in, dim_out, words,
                  epsilon, 0.f, scale};
    if (!faith::dual_exponent(q, &a.qv)) {
        faith::set_error("faith_softmax_verification: q=%d is neither FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF nor the bits of an "
                         "exponent in (1, inf)", q);
        return FAITH_ERR_UNSUPPORTED;
    }
    const bool vec4 = dim_out % 4 == 0 && faith::aligned(src_lw, 16) && faith::aligned(src_uw, 16) &&
                      faith::aligned(out_lw, 16) && faith::aligned(out_uw, 16);
    hipStream_t st = static_cast<hipStream_t>(stream);
    bool ok;
    switch (q) {
        case FAITH_Q_1: ok = dispatch<FAITH_Q_1>(a, vec4, st); break;
        case FAITH_Q_2: ok = dispatch<FAITH_Q_2>(a, vec4, st); break;
        case FAITH_Q_INF: ok = dispatch<FAITH_Q_INF>(a, vec4, st); break;
        default: ok = dispatch<Q_GENERAL>(a, vec4, st); break;
    }
    if (!ok) {
        faith::set_error("faith_softmax_verification: a [dim_in=%d, dim_out=%d] slab does not fit the registers (see "
                         "faith_softmax_fits) or, with many perturbed words, the 160 KB of LDS of one workgroup; compose exp, row sum, reciprocal and multiply instead",
                         dim_in, dim_out);
        return FAITH_ERR_UNSUPPORTED;
    }
    return faith::check_launch("faith_softmax_verification");
}

// 1 if faith_softmax_verification takes this slab (given 16-byte aligned tensors), 0 if the caller has to compose
// the four operators.
extern "C" int faith_softmax_fits(int dim_in, int dim_out) {
    if (dim_in <= 0 || dim_out <= 0) return 0;
    const int vec = dim_out % 4 == 0 ? 4 : 1;
    int tpr = 1;
    while (tpr * vec < dim_out) tpr <<= 1;
    if (tpr > WAVE) return 0;
    return vec == 4 ? (1024 / tpr) * 8 >= dim_in : (1024 / tpr) * 24 >= dim_in;
}

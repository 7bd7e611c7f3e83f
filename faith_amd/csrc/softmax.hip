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

// Buffer addressing: the hardware compares thread offset + uniform offset against the window's size; accesses at
// or beyond it return zero (loads) or are dropped (stores).
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t slab_window(const float *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(base), 0, (int)bytes, 0x00020000);
}
// One butterfly step at distance m for 2 N values through the LDS crossbar, the 2 N exchanges in flight together.
// (The swap instructions v_permlane16_swap / v_permlane32_swap do distances 16 and 32 on the vector ALU, but with
// the copies and wait states they need they measured slower here: 63.7 against 61.8 us on a [256 x 128] slab.)
template <int Q, int N>
__device__ __forceinline__ void combine_across(float (&a)[N], float (&b)[N], int m) {
    float ta[N], tb[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        ta[i] = __shfl_xor(a[i], m, WAVE);
        tb[i] = __shfl_xor(b[i], m, WAVE);
    }
#pragma unroll
    for (int i = 0; i < N; ++i) {
        a[i] = ncomb<Q>(a[i], ta[i]);
        b[i] = ncomb<Q>(b[i], tb[i]);
    }
}
template <int VEC>
__device__ __forceinline__ Vec<VEC> slab_load(__amdgpu_buffer_rsrc_t w, unsigned thread_off, unsigned uniform_off) {
    Vec<VEC> d;
    if constexpr (VEC == 4) {
        const uintx4 t = __builtin_amdgcn_raw_buffer_load_b128(w, thread_off, uniform_off, 0);
        d.v = make_float4(__uint_as_float(t.x), __uint_as_float(t.y), __uint_as_float(t.z), __uint_as_float(t.w));
    } else {
        d.v = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(w, thread_off, uniform_off, 0));
    }
    return d;
}
template <int VEC>
__device__ __forceinline__ void slab_store(const Vec<VEC> &d, __amdgpu_buffer_rsrc_t w, unsigned thread_off, unsigned uniform_off) {
    if constexpr (VEC == 4) {
        const uintx4 t = {__float_as_uint(d.v.x), __float_as_uint(d.v.y), __float_as_uint(d.v.z), __float_as_uint(d.v.w)};
        __builtin_amdgcn_raw_buffer_store_b128(t, w, thread_off, uniform_off, 2 /* non-temporal */);
    } else {
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(d.v), w, thread_off, uniform_off, 2);
    }
}

// Four wavefronts per SIMD (128 registers): two workgroups of 512 threads or four of 256 on a CU, so that one's
// arithmetic runs beside another's loads and stores.  (A general exponent keeps the registers it needs.)
template <int Q, int VEC, int NTHREADS, int RPT>
__global__ void __launch_bounds__(NTHREADS, (Q == Q_GENERAL && NTHREADS < 1024) ? 1 : 4) softmax_kernel(const SoftmaxArgs a, const int tpr_log2) {
    // the scalar arguments as locals (read through the argument block inside the lambdas below, the block was
    // copied to private memory in the instantiations for a general exponent)
    const int n_words = a.words;
    const float dual_q = a.qv;
    const float eps_v = a.eps;
    const int d_in = a.D;
    const int d_out = a.H;
    const float scale_v = a.scale;
    constexpr int NW = NTHREADS / WAVE;
    extern __shared__ float smem[];
    const int TPR = 1 << tpr_log2, TH = TPR * VEC, RG = NTHREADS >> tpr_log2;
    float *part = smem;                              // [words][NW][2][TH] column partial norms (x, then e)
    float *col = part + n_words * NW * 2 * TH;       // [5][TH]: k_lo, k_up of exp; e.lb, e.ub; b = l_e
    float *spart = col + 5 * TH;                     // [words][NW][2] partial norms of the one-neuron objects s, r
    float *scal = spart + n_words * NW * 2;          // [2]: s.lb, s.ub

    const int r = blockIdx.x;
    const int tid = threadIdx.x, lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid & (TPR - 1), rg = tid >> tpr_log2;
    const int col0 = c * VEC;
    const bool col_ok = col0 < d_out;                  // VEC == 4: H % 4 == 0, so the four columns stand or fall together
    const int blk = d_in / n_words;

    // the column's constant terms first: they are needed right after the first barrier and would otherwise
    // be fetched then, behind the whole machine's slab loads
    const size_t bi = (size_t)r * d_out + tid;         // thread h < H speaks for column h
    float xlb = 0.f, xub = 0.f;
    if (tid < d_out) {
        xlb = a.lb[bi];
        xub = a.ub[bi];
    }

    // ---- x: the slab into registers
    // Buffer addressing over the row's own slab: a thread whose column does not exist is sent outside the window
    // and slab rows past D_in fall outside it, where loads return zero and stores are dropped -- no branch and
    // no wait between the loads, all 2 RPT of a thread are in flight together.
    const unsigned slab_bytes = (unsigned)d_in * d_out * 4u;
    const size_t slab0 = (size_t)r * d_in * d_out;
    const unsigned voff = col_ok ? ((unsigned)rg * d_out + col0) * 4u : 0x80000000u;
    const unsigned step_bytes = (unsigned)RG * d_out * 4u;
    Vec<VEC> dl[RPT], du[RPT];
    {
        const __amdgpu_buffer_rsrc_t wl = slab_window(a.lw + slab0, slab_bytes), wu = slab_window(a.uw + slab0, slab_bytes);
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            dl[i] = slab_load<VEC>(wl, voff, i * step_bytes);
            du[i] = slab_load<VEC>(wu, voff, i * step_bytes);
        }
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {        // one rounding, as the separate scaling stores it
                dl[i].set(v, dl[i].get(v) * scale_v);
                du[i].set(v, du[i].get(v) * scale_v);
            }
        }
    }

    // column norms of what dl / du hold -> part; the caller synchronises
    // A perturbed word owns `blk` consecutive rows.  When blk is a multiple of RG, the rows i * RG + rg of step i
    // belong to one word for every thread: the membership test is then a scalar one per step instead of one per
    // value (the usual case; rows past D_in hold zeros and add nothing to any norm).
    const bool whole_steps = blk % RG == 0;
    const int steps_per_word = blk / RG;
    auto column_norms = [&]() __attribute__((always_inline)) {
        for (int w = 0; w < n_words; ++w) {
            const int lo_row = w * blk, hi_row = lo_row + blk;
            float pl[VEC], pu[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v) pl[v] = pu[v] = 0.f;
            if (whole_steps) {
                const int lo_i = w * steps_per_word, hi_i = lo_i + steps_per_word;
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    if (i >= lo_i && i < hi_i) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            float xl = dl[i].get(v), xu = du[i].get(v);
                            // (general exponent: opaque copies as below, or log |x| of all 2 RPT VEC values is formed
                            // outside the loop over the words and held)
                            if (Q == Q_GENERAL) asm volatile("" : "+v"(xl), "+v"(xu));
                            pl[v] = nacc<Q>(pl[v], xl, dual_q);
                            pu[v] = nacc<Q>(pu[v], xu, dual_q);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    const int row = i * RG + rg;
                    if (row >= lo_row && row < hi_row) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            // opaque copies: |x| or x^2 of every value would otherwise be formed once, outside the
                            // loop over the words, and held (64 more registers)
                            float xl = dl[i].get(v), xu = du[i].get(v);
                            asm volatile("" : "+v"(xl), "+v"(xu));
                            pl[v] = nacc<Q>(pl[v], xl, dual_q);
                            pu[v] = nacc<Q>(pu[v], xu, dual_q);
                        }
                    }
                }
            }
            for (int m = TPR; m < WAVE; m <<= 1) combine_across<Q>(pl, pu, m);
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
    auto neuron_norms = [&]() __attribute__((always_inline)) {
        for (int w = 0; w < n_words; ++w) {
            const int lo_row = w * blk, hi_row = lo_row + blk;
            float pl[1] = {0.f}, pu[1] = {0.f};
            if (c == 0) {
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    const int row = i * RG + rg;
                    if (row >= lo_row && row < hi_row) {
                        pl[0] = nacc<Q>(pl[0], sl[i], dual_q);
                        pu[0] = nacc<Q>(pu[0], su[i], dual_q);
                    }
                }
            }
            // the lanes that hold something are TPR apart: the butterfly starts there
            for (int m = TPR; m < WAVE; m <<= 1) combine_across<Q>(pl, pu, m);
            if (lane == 0) {
                spart[(w * NW + wv) * 2 + 0] = pl[0];
                spart[(w * NW + wv) * 2 + 1] = pu[0];
            }
        }
    };
    // [lb - eps * sum of norms, ub + eps * sum of norms] from partial norms (Bounds.py:311-326)
    auto interval = [&](const float *p, int stride, int offset, float lb, float ub, float &l, float &u) __attribute__((always_inline)) {
        l = lb;
        u = ub;
        for (int w = 0; w < n_words; ++w) {
            // the wavefronts' partial norms are fetched eight at a time before the first is used: one LDS latency
            // per eight wavefronts instead of one per wavefront (combined in the order of the wavefronts all the same)
            constexpr int CH = NW < 8 ? NW : 8;
            float nl = 0.f, nu = 0.f;
#pragma unroll
            for (int g0 = 0; g0 < NW; g0 += CH) {
                float vl[CH], vu[CH];
#pragma unroll
                for (int g = 0; g < CH; ++g) {
                    vl[g] = p[((w * NW + g0 + g) * 2 + 0) * stride + offset];
                    vu[g] = p[((w * NW + g0 + g) * 2 + 1) * stride + offset];
                }
#pragma unroll
                for (int g = 0; g < CH; ++g) {
                    nl = ncomb<Q>(nl, vl[g]);
                    nu = ncomb<Q>(nu, vu[g]);
                }
            }
            l += (-eps_v) * nfin<Q>(nl, dual_q);
            u += eps_v * nfin<Q>(nu, dual_q);
        }
    };

    // the same for a one-neuron object from spart, every thread for itself: lane g takes wavefront g's partial norm
    // and a butterfly over NW lanes combines them (2 log2 NW exchanges per word instead of 2 NW reads and sums)
    auto neuron_interval = [&](float lb, float ub, float &l, float &u) __attribute__((always_inline)) {
        l = lb;
        u = ub;
        for (int w = 0; w < n_words; ++w) {
            float nl = spart[(w * NW + lane % NW) * 2 + 0], nu = spart[(w * NW + lane % NW) * 2 + 1];
#pragma unroll
            for (int m = 1; m < NW; m <<= 1) {
                nl = ncomb<Q>(nl, __shfl_xor(nl, m, WAVE));
                nu = ncomb<Q>(nu, __shfl_xor(nu, m, WAVE));
            }
            l += (-eps_v) * nfin<Q>(nl, dual_q);
            u += eps_v * nfin<Q>(nu, dual_q);
        }
    };

    // ---- e = exp(x): Bounds.py:970-1003
    column_norms();
    __syncthreads();
    if (tid < d_out) {
        xlb *= scale_v;
        xub *= scale_v;
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
        sl[i] = tl;
        su[i] = tu;
    }
    // The butterfly over the threads of a slab row, all RPT rows per step.  Distances 1 to 8 are lane permutations
    // inside a row of 16 lanes, which the vector ALU does on its own operand (no trip through the LDS crossbar):
    // 1 and 2 as permutations of four lanes; after them the four lanes of a group hold one value, so mirroring
    // eight lanes fetches what lane ^ 4 holds, and after that mirroring sixteen fetches what lane ^ 8 holds.
    // Longer distances go through the crossbar, 2 RPT exchanges in flight at a time.
    auto butterfly_step = [&](auto exchange) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            sl[i] += exchange(sl[i]);
            su[i] += exchange(su[i]);
        }
    };
    if (TPR > 1) butterfly_step([](float x) { return lane_permute<0xB1>(x); });      // lanes 1 0 3 2
    if (TPR > 2) butterfly_step([](float x) { return lane_permute<0x4E>(x); });      // lanes 2 3 0 1
    if (TPR > 4) butterfly_step([](float x) { return lane_permute<0x141>(x); });     // eight lanes mirrored
    if (TPR > 8) butterfly_step([](float x) { return lane_permute<0x140>(x); });     // sixteen lanes mirrored
    for (int m = 16; m < TPR; m <<= 1) combine_across<FAITH_Q_1>(sl, su, m);      // Q_1: a sum
    if (wv == 0) {
        float tl = 0.f, tu = 0.f;
        for (int h = lane; h < d_out; h += WAVE) {
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
        neuron_interval(slb, sub, l, u);
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
    neuron_interval(rlb, rub, al, au);
    if (tid < d_out) {
        const float elb = col[2 * TH + tid], eub = col[3 * TH + tid];
        float bt, unused;
        interval(part, TH, tid, elb, eub, bt, unused);
        col[4 * TH + tid] = bt;
        const float gl = -al * bt, gu = -au * bt;
        a.olb[bi] = ((al > 0.f ? elb : eub) * al + gl) + (bt > 0.f ? rlb : rub) * bt;
        a.oub[bi] = ((au > 0.f ? eub : elb) * au + gu) + (bt > 0.f ? rub : rlb) * bt;
    }
    __syncthreads();
    float bt[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) bt[v] = col[4 * TH + col0 + v];
    const __amdgpu_buffer_rsrc_t wol = slab_window(a.olw + slab0, slab_bytes), wou = slab_window(a.ouw + slab0, slab_bytes);
    // a_l and a_u are one neuron's bounds, the same for the whole workgroup: both positive (a reciprocal of a
    // positive sum) is the case that runs without the selects on their sign
    if (al > 0.f && au > 0.f) {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            Vec<VEC> ol, ou;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                ol.set(v, dl[i].get(v) * al + (bt[v] > 0.f ? sl[i] : su[i]) * bt[v]);
                ou.set(v, du[i].get(v) * au + (bt[v] > 0.f ? su[i] : sl[i]) * bt[v]);
            }
            slab_store<VEC>(ol, wol, voff, i * step_bytes);
            slab_store<VEC>(ou, wou, voff, i * step_bytes);
        }
    } else {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            Vec<VEC> ol, ou;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float el = dl[i].get(v), eu = du[i].get(v);
                ol.set(v, (al > 0.f ? el : eu) * al + (bt[v] > 0.f ? sl[i] : su[i]) * bt[v]);
                ou.set(v, (au > 0.f ? eu : el) * au + (bt[v] > 0.f ? su[i] : sl[i]) * bt[v]);
            }
            slab_store<VEC>(ol, wol, voff, i * step_bytes);
            slab_store<VEC>(ou, wou, voff, i * step_bytes);
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
        if ((512 / tpr) * 8 >= a.D) return launch<Q, 4, 512, 8>(a, k, st);
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

// Concretization and the ReLU / tanh relaxations, each as ONE pass over HBM.
//
// Arithmetic follows the reference's PyTorch Bounds methods
// (Transformer_Verification_Code/Verifiers/Bounds.py:311-326 concretize, :348-381 new /
// add_linear, :921-963 ori_relu, :1027-1103 ori_tanh), not its CUDA kernels, which hard-wire
// q = 2 and differ at the branch boundaries.
//
// Natural layout [rows, D_in, H] (the layout the reference's Python keeps its tensors in):
//   a workgroup owns one row r and a tile of TH neighbouring neurons.  Lanes run along H, so
//   every global access is a run of TH*4 contiguous bytes; the D_in rows of the tile are spread
//   over the workgroup's threads and stay in registers between the norm reduction and the
//   scaling, so lw / uw are read once and lw' / uw' written once.
//   Per thread: partial q-norms of its rows -> LDS -> one thread per neuron finishes the norm,
//   forms [l, u], derives the two lines (slope k, anchor x0, offset y0) -> LDS -> every thread
//   scales what it holds and stores it.
//
// Transposed layout [rows, H, D_in] (what the reference's CUDA adapters hand over,
// Bounds.py:1210-1211): D_in is contiguous, a wavefront owns a neuron and reduces with
// cross-lane shuffles.
//
// This file is built with -ffp-contract=off: the reference rounds (b - x0) * k and the
// following + y0 separately, and l = lb + (-eps * norm) likewise.
#include "relax_lines.h"

namespace {

struct ActArgs {
    const float *lb, *ub, *lw, *uw;
    float *olb, *oub, *olw, *ouw;
    float *l, *u;
    int rows, D, H, words;
    float eps;
    // optional second bound object of the same D (concretize only): one launch covers both
    const float *lb2 = nullptr, *ub2 = nullptr, *lw2 = nullptr, *uw2 = nullptr;
    float *l2 = nullptr, *u2 = nullptr;
    int rows2 = 0, H2 = 0;
    float qv = 0.f;     // the dual exponent when it is none of 1, 2, inf
    int cached_stores = 0;   // general kernel: results through the L2 as ordinary stores (rows that share 64-byte sectors)
    int remap = 0;      // order of the tiles (register-resident kernels): 0 as numbered, 1 an eighth of the range per XCD, 2 whole rows per XCD
};

// ------------------------------------------------------------------ natural layout
// exp-based pieces for the tanh lines, all in double: with t = exp(2x),
// tanh x = (t - 1) / (t + 1) and 1 / cosh^2 x = 4 t / (t + 1)^2.  |x| is clamped at 20, where
// tanh is 1 to 17 digits.
struct TanhAt {
    double th, s2;
};
__device__ __forceinline__ TanhAt tanh_at(float x) {
    const double t = exp(2.0 * fmin(fmax((double)x, -20.0), 20.0));
    const double r = 1.0 / (t + 1.0);
    return {(t - 1.0) * r, 4.0 * t * r * r};
}

// Tangent point search of Bounds.py:1065-1075 (lower = true) and :1082-1092 (lower = false): the ten bisection
// steps, in fp32 as the reference takes them on its fp32 tensors.  `anchor` is the far end of the interval (u for
// the lower line, l for the upper line).  The reference asks whether (tanh difference) / (distance) - sech^2(d) is
// positive; the distance (+1e-12) is positive, and so is (t + 1)^2 with t = exp(2 d), tanh d = (t - 1) / (t + 1),
// sech^2 d = 4 t / (t + 1)^2, so the sign is that of
//     (tanh(anchor) (t + 1) - (t - 1)) (t + 1) - 4 t distance          (lower; the upper line with the first factor negated)
// -- no division, one exponential, fourteen instructions a step: the chain of ten dependent steps is what a tile
// waits for.  A sign that differs from the quotient form's can only occur where the quantity is within rounding of
// zero, i.e. at the tangent point itself, where the slope of the line is stationary.
template <bool LOWER>
__device__ __forceinline__ float tanh_tangent_point(float l, float u) {
    constexpr float TWO_LOG2E = 2.885390081777926815f;
    const float ea = __builtin_amdgcn_exp2f(__builtin_amdgcn_fmed3f(LOWER ? u : l, -20.f, 20.f) * TWO_LOG2E);
    const float ta = (ea - 1.f) / (ea + 1.f);
    float d = (LOWER ? l : u) / 2, a = LOWER ? l : 0.f, b = LOWER ? 0.f : u;
#pragma unroll
    for (int it = 0; it < 10; ++it) {
        const float t = __builtin_amdgcn_exp2f(__builtin_amdgcn_fmed3f(d, -20.f, 20.f) * TWO_LOG2E);
        const float p = t + 1.f, tm1 = t - 1.f;
        const float c4 = __builtin_fmaf(LOWER ? u - d : d - l, 4.f, 4.f * TINY);
        const float q = LOWER ? __builtin_fmaf(ta, p, -tm1) : __builtin_fmaf(-ta, p, tm1);
        const bool go = __builtin_fmaf(q, p, -(t * c4)) > 0.f;
        if (LOWER == go)     // lower & v > 0, or upper & v <= 0: move right
            a = d;
        else                 // move left
            b = d;
        d = (a + b) / 2;     // the end that moved is d: (d + b) / 2 or (d + a) / 2
    }
    return d;
}

// The line through the tangent point found and the anchor, formed in double; `ta` = tanh(anchor).
template <bool LOWER>
__device__ __forceinline__ Line tanh_tangent_line(float l, float u, float d, double ta) {
    const double td = tanh_at(d).th;
    if (LOWER) return {(float)((td - ta) / (double)((d - u) + TINY)), d, (float)td};
    return {(float)((td - ta) / (double)((d - l) + TINY)), d, (float)td};
}

// One-signed interval: tangent at the midpoint and chord (Bounds.py:1037-1060).
__device__ __forceinline__ void tanh_pure_lines(float l, float u, Line &lo, Line &up) {
    const float m = (l + u) / 2;
    const TanhAt fm = tanh_at(m);
    const double tl = tanh_at(l).th, tu = tanh_at(u).th;
    const Line tangent = {(float)fm.s2, m, (float)fm.th};
    const Line chord = {(float)((tu - tl) / (double)((u - l) + TINY)), l, (float)tl};
    if (u < 0.f) {
        lo = tangent;
        up = chord;
    } else {
        lo = chord;
        up = tangent;
    }
}

// tanh lines of the TH neurons of a tile whose concrete intervals are in s_lu ([2][TH]), entered by
// every thread after a barrier: four wavefronts share the per-neuron work, lane = neuron.  Slopes end
// up in s_ln[0 .. TH) and s_ln[3 TH .. 4 TH) (complete once the barriers inside have been passed), the
// constant terms in olb / oub.
template <int TH>
__device__ __forceinline__ void tanh_stage(const ActArgs &a, const float *s_lu, float *s_ln, float lb, float ub, size_t bi,
                                           bool n_ok, int lane, int wv) {
    // 0 = lower tangent search, 1 = upper tangent search (straddling neurons), 2 = tangent / chord of one-signed
    // neurons, 3 = tanh of both ends in double, which the lines of the straddling neurons pass through: the
    // searches do not wait for it
    __shared__ double s_anchor[2 * TH];
    float l = 0.f, u = 0.f, d = 0.f;
    bool searched = false;
    if (wv < 4 && n_ok) {
        l = s_lu[lane];
        u = s_lu[TH + lane];
        const bool pure = (u < 0.f || l > 0.f);
        if (wv == 2) {
            if (pure) {
                Line lo, up;
                tanh_pure_lines(l, u, lo, up);
                s_ln[lane] = lo.k; s_ln[TH + lane] = lo.x0; s_ln[2 * TH + lane] = lo.y0;
                s_ln[3 * TH + lane] = up.k; s_ln[4 * TH + lane] = up.x0; s_ln[5 * TH + lane] = up.y0;
            }
        } else if (!pure) {
            if (wv == 3) {
                s_anchor[lane] = tanh_at(u).th;
                s_anchor[TH + lane] = tanh_at(l).th;
            } else {
                searched = true;
                d = wv == 0 ? tanh_tangent_point<true>(l, u) : tanh_tangent_point<false>(l, u);
            }
        }
    }
    __syncthreads();
    if (searched) {
        if (wv == 0) {
            const Line lo = tanh_tangent_line<true>(l, u, d, s_anchor[lane]);
            s_ln[lane] = lo.k; s_ln[TH + lane] = lo.x0; s_ln[2 * TH + lane] = lo.y0;
        } else {
            const Line up = tanh_tangent_line<false>(l, u, d, s_anchor[TH + lane]);
            s_ln[3 * TH + lane] = up.k; s_ln[4 * TH + lane] = up.x0; s_ln[5 * TH + lane] = up.y0;
        }
    }
    __syncthreads();
    if (wv == 0 && n_ok) {
        const Line lo = {s_ln[lane], s_ln[TH + lane], s_ln[2 * TH + lane]};
        const Line up = {s_ln[3 * TH + lane], s_ln[4 * TH + lane], s_ln[5 * TH + lane]};
        a.olb[bi] = line_bias(lo, lb, ub);
        a.oub[bi] = line_bias(up, ub, lb);
    }
}

// The per-neuron part of a natural-layout tile, entered by every thread after the partial norms are
// in `part` ([words][NW][2][TH]) and a barrier: one lane per neuron (wavefront 0) finishes the
// norms and concretizes; the slopes of the two lines end up in s_ln[0 .. TH) and s_ln[3 TH .. 4 TH),
// the constant terms in olb / oub.  Ends with a barrier (except for CONCRETIZE).
// lb0 / ub0: the neuron's constant terms (lanes of wavefront 0 with n_ok), which the caller fetches before it
// loads its coefficients: fetched here they would be one more memory latency between the loads and the stores of
// every tile.
template <int MODE, int Q, int NW, int TH>
__device__ __forceinline__ void neuron_stage(const ActArgs &a, const float *part, float *s_lu, float *s_ln, float lb0,
                                             float ub0, float *__restrict__ p_l, float *__restrict__ p_u, size_t bi,
                                             bool n_ok, int lane, int wv) {
    if (wv == 0 && n_ok) {
        float l = lb0, u = ub0;
        for (int w = 0; w < a.words; ++w) {
            float nl = 0.f, nu = 0.f;
#pragma unroll
            for (int g = 0; g < NW; ++g) {
                nl = ncomb<Q>(nl, part[((w * NW + g) * 2 + 0) * TH + lane]);
                nu = ncomb<Q>(nu, part[((w * NW + g) * 2 + 1) * TH + lane]);
            }
            l += (-a.eps) * nfin<Q>(nl, a.qv);
            u += a.eps * nfin<Q>(nu, a.qv);
        }
        if (p_l) p_l[bi] = l;
        if (p_u) p_u[bi] = u;
        if (MODE != TANH && MODE != CONCRETIZE) {
            float klo, kup, olb, oub;
            relax_point<MODE>(l, u, lb0, ub0, klo, kup, olb, oub);
            s_ln[lane] = klo;
            s_ln[3 * TH + lane] = kup;
            a.olb[bi] = olb;
            a.oub[bi] = oub;
        } else if (MODE == TANH) {
            s_lu[lane] = l;
            s_lu[TH + lane] = u;
        }
    }
    if (MODE == CONCRETIZE) return;
    __syncthreads();

    if (MODE == TANH) tanh_stage<TH>(a, s_lu, s_ln, lb0, ub0, bi, n_ok, lane, wv);
}

// TPR threads cover one row of the tile (TH = TPR * VEC neurons); RG = NTHREADS / TPR rows are
// in flight per step; a thread keeps RPT rows.  D_in <= RG * RPT is the register-resident case;
// larger D_in is walked in chunks and read a second time for the scaling.
template <int MODE, int Q, int VEC, int TPR, int NTHREADS, int RPT>
__global__ void __launch_bounds__(NTHREADS) act_natural(const ActArgs a) {
    constexpr int TH = TPR * VEC;
    constexpr int RG = NTHREADS / TPR;
    constexpr int NW = NTHREADS / WAVE;
    static_assert(TH <= WAVE && TPR <= WAVE && NW >= 4, "per-neuron stages use one lane per neuron in wavefronts 0 ... 3");
    extern __shared__ float smem[];
    float *part = smem;                       // [words][NW][2][TH] per-wavefront partial norms
    float *s_lu = part + a.words * NW * 2 * TH;   // [2][TH] concrete interval
    float *s_ln = s_lu + 2 * TH;              // [2][3][TH] lower / upper line (k, x0, y0)

    // concretize only: a second bound object of the same dim_in (its own dim_out) in the same launch
    const int tiles1 = (a.H + TH - 1) / TH;
    const bool second = MODE == CONCRETIZE && (int)blockIdx.x >= a.rows * tiles1;
    const int H = second ? a.H2 : a.H;
    const int tiles = (H + TH - 1) / TH;
    int bid = second ? blockIdx.x - a.rows * tiles1 : blockIdx.x;
    if (a.remap == 2) {
        // whole rows of an object dealt to the XCDs (workgroup w runs on XCD w % 8; the launcher has checked that
        // both objects start on a multiple of 8 and have a multiple of 8 rows)
        const int idx = bid / 8, x = bid % 8;
        bid = (idx / tiles * 8 + x) * tiles + idx % tiles;
    }
    const float *__restrict__ p_lw = second ? a.lw2 : a.lw, *__restrict__ p_uw = second ? a.uw2 : a.uw;
    const float *__restrict__ p_lb = second ? a.lb2 : a.lb, *__restrict__ p_ub = second ? a.ub2 : a.ub;
    float *__restrict__ p_l = second ? a.l2 : a.l, *__restrict__ p_u = second ? a.u2 : a.u;
    const int r = bid / tiles;
    const int col0 = (bid % tiles) * TH;
    const int tid = threadIdx.x;
    const int lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid % TPR, rg = tid / TPR;
    const int col = col0 + c * VEC;
    const bool col_ok = col < H;
    const size_t base = (size_t)r * a.D * H + col;
    const int blk = a.D / a.words;
    constexpr int CHUNK = RG * RPT;
    const int nchunks = (a.D + CHUNK - 1) / CHUNK;

    const int column = col0 + lane;
    const bool n_ok = lane < TH && column < H;
    const size_t bi = (size_t)r * H + column;
    float lb0 = 0.f, ub0 = 0.f;
    if (wv == 0 && n_ok) {
        lb0 = p_lb[bi];
        ub0 = p_ub[bi];
    }

    Vec<VEC> dl[RPT], du[RPT];
    // concretize only: an upper interval nobody asked for (the first operand of a dot product: its planes
    // take x from below on both sides) -- the upper coefficients then stay where they are
    const bool want_u = MODE != CONCRETIZE || p_u != nullptr;

    if (nchunks > 1 && lane < TPR) {
        for (int w = 0; w < a.words; ++w)
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                part[((w * NW + wv) * 2 + 0) * TH + c * VEC + v] = 0.f;
                part[((w * NW + wv) * 2 + 1) * TH + c * VEC + v] = 0.f;
            }
    }

    for (int ch = 0; ch < nchunks; ++ch) {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int row = ch * CHUNK + i * RG + rg;
            if (col_ok && row < a.D) {
                dl[i].load(p_lw + base + (size_t)row * H);
                if (want_u) du[i].load(p_uw + base + (size_t)row * H);
                else du[i].zero();
            } else {
                dl[i].zero();
                du[i].zero();
            }
        }
        for (int w = 0; w < a.words; ++w) {
            const int lo_row = w * blk, hi_row = lo_row + blk;
            float pl[VEC], pu[VEC];
#pragma unroll
            for (int v = 0; v < VEC; ++v) pl[v] = pu[v] = 0.f;
            if (blk % RG == 0) {
                // a word owns a whole number of steps (RG rows each): whether step ch * RPT + i counts for it is a
                // scalar test per step instead of one per value (see resident_partials)
                const int lo_s = w * (blk / RG) - ch * RPT, hi_s = lo_s + blk / RG;
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    if (i >= lo_s && i < hi_s) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            pl[v] = nacc<Q>(pl[v], dl[i].get(v), a.qv);
                            pu[v] = nacc<Q>(pu[v], du[i].get(v), a.qv);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int i = 0; i < RPT; ++i) {
                    const int row = ch * CHUNK + i * RG + rg;
                    if (row >= lo_row && row < hi_row) {
#pragma unroll
                        for (int v = 0; v < VEC; ++v) {
                            float xl = dl[i].get(v), xu = du[i].get(v);
                            asm volatile("" : "+v"(xl), "+v"(xu));      // keeps |x| from being formed outside the word loop and held
                            pl[v] = nacc<Q>(pl[v], xl, a.qv);
                            pu[v] = nacc<Q>(pu[v], xu, a.qv);
                        }
                    }
                }
            }
            // lanes of one wavefront that share a column: butterfly over the row groups
            combine_from<Q, TPR>(pl, pu);
            if (lane < TPR) {
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    float *sl = &part[((w * NW + wv) * 2 + 0) * TH + c * VEC + v];
                    float *su = &part[((w * NW + wv) * 2 + 1) * TH + c * VEC + v];
                    if (nchunks > 1) {
                        *sl = ncomb<Q>(*sl, pl[v]);
                        *su = ncomb<Q>(*su, pu[v]);
                    } else {
                        *sl = pl[v];
                        *su = pu[v];
                    }
                }
            }
        }
    }
    __syncthreads();

    neuron_stage<MODE, Q, NW, TH>(a, part, s_lu, s_ln, lb0, ub0, p_l, p_u, bi, n_ok, lane, wv);
    if (MODE == CONCRETIZE) return;

    if (!col_ok) return;
    float klo[VEC], kup[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        klo[v] = s_ln[c * VEC + v];
        kup[v] = s_ln[3 * TH + c * VEC + v];
    }
    // rows that do not start on 64-byte boundaries: a tile's row segments share their first and last 64 bytes with
    // the neighbouring tiles'; streamed past the cache, each part would be a partial write to memory
    const bool split_sectors = a.cached_stores != 0;
    for (int ch = 0; ch < nchunks; ++ch) {
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const int row = ch * CHUNK + i * RG + rg;
            if (row < a.D) {
                const size_t off = base + (size_t)row * H;
                if (nchunks > 1) {
                    dl[i].load(p_lw + off);
                    du[i].load(p_uw + off);
                }
                Vec<VEC> ol, ou;
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    const float xl = dl[i].get(v), xu = du[i].get(v);
                    ol.set(v, (klo[v] > 0.f ? xl : xu) * klo[v]);
                    ou.set(v, (kup[v] > 0.f ? xu : xl) * kup[v]);
                }
                if (split_sectors) {
                    ol.store_cached(a.olw + off);
                    ou.store_cached(a.ouw + off);
                } else {
                    ol.store(a.olw + off);
                    ou.store(a.ouw + off);
                }
            }
        }
    }
}

// Column partial norms of a register-resident tile (thread (c, rg) holds rows i * RG + rg, i < RPT, of VEC columns)
// -> part[words][NW][2][TH].  A perturbed word owns D_in / words consecutive rows; when that is a multiple of RG the
// rows of step i belong to one word for every thread, and whether a step counts for a word is a scalar test per
// step instead of a test (and a masked accumulation) per value -- for a general exponent, whose accumulation is two
// quarter-rate instructions per value, that halves the arithmetic of a two-word tile.
template <int Q, int VEC, int RPT, int RG, int TPR, int NW, int TH>
__device__ __forceinline__ void resident_partials(const ActArgs &a, const Vec<VEC> (&dl)[RPT], const Vec<VEC> (&du)[RPT],
                                                  float *part, int rg, int c, int lane, int wv) {
    const int blk = a.D / a.words;
    const bool whole_steps = blk % RG == 0;
    const int steps = blk / RG;
    for (int w = 0; w < a.words; ++w) {
        float pl[VEC], pu[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) pl[v] = pu[v] = 0.f;
        if (whole_steps) {
            const int lo_i = w * steps, hi_i = lo_i + steps;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                if (i >= lo_i && i < hi_i) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        pl[v] = nacc<Q>(pl[v], dl[i].get(v), a.qv);
                        pu[v] = nacc<Q>(pu[v], du[i].get(v), a.qv);
                    }
                }
            }
        } else {
            const int lo_row = w * blk, hi_row = lo_row + blk;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                const int row = i * RG + rg;
                if (row >= lo_row && row < hi_row) {
#pragma unroll
                    for (int v = 0; v < VEC; ++v) {
                        // opaque copies: |x| (or its logarithm) of every value would otherwise be formed once,
                        // outside the loop over the words, and held: 64 more registers
                        float xl = dl[i].get(v), xu = du[i].get(v);
                        asm volatile("" : "+v"(xl), "+v"(xu));
                        pl[v] = nacc<Q>(pl[v], xl, a.qv);
                        pu[v] = nacc<Q>(pu[v], xu, a.qv);
                    }
                }
            }
        }
        combine_from<Q, TPR>(pl, pu);
        if (lane < TPR) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                part[((w * NW + wv) * 2 + 0) * TH + c * VEC + v] = pl[v];
                part[((w * NW + wv) * 2 + 1) * TH + c * VEC + v] = pu[v];
            }
        }
    }
}

// The common shape of the natural layout, straight-line: D_in <= RG * RPT (everything a thread
// loads stays in registers), D_in a multiple of RG and H a multiple of the tile width, 16-byte
// aligned.  Whether a row exists is then the same for every thread (a scalar branch), there are no
// column predicates and no second pass, and the kernel is a slab copy with the reduction and the
// per-neuron stage between its loads and its stores: at configuration 1 it runs within 3 % of
// that copy, where the general kernel above needs 25 % more.
template <int MODE, int Q, int TPR, int NTHREADS, int RPT, int WPE = 4, bool NTL = false, int MAXW = 8>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(WPE, MAXW))) act_resident(const ActArgs a) {
    constexpr int VEC = 4, TH = TPR * VEC, RG = NTHREADS / TPR, NW = NTHREADS / WAVE;
    static_assert(TH <= WAVE && NW >= 4, "per-neuron stages use one lane per neuron in wavefronts 0 ... 3");
    extern __shared__ float smem[];
    float *part = smem;                           // [words][NW][2][TH] per-wavefront partial norms
    float *s_lu = part + a.words * NW * 2 * TH;   // [2][TH] concrete interval
    float *s_ln = s_lu + 2 * TH;                  // [2][3][TH] lower / upper line (k, x0, y0)

    const int tiles = a.H / TH;
    int bid = blockIdx.x;
    // workgroup w runs on XCD w % 8
    if (a.remap == 1) bid = (int)(blockIdx.x % 8) * (int)(gridDim.x / 8) + (int)(blockIdx.x / 8);
    if (a.remap == 2) {
        const int idx = (int)(blockIdx.x / 8), x = (int)(blockIdx.x % 8);
        bid = (idx / tiles * 8 + x) * tiles + idx % tiles;
    }
    const int r = bid / tiles, col0 = (bid % tiles) * TH;
    const int tid = threadIdx.x, lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid % TPR, rg = tid / TPR;
    const size_t base = ((size_t)r * a.D + rg) * a.H + col0 + c * VEC;
    const size_t row_step = (size_t)RG * a.H;
    const float *__restrict__ p_lw = a.lw + base, *__restrict__ p_uw = a.uw + base;
    const size_t bi = (size_t)r * a.H + col0 + lane;
    float lb0 = 0.f, ub0 = 0.f;
    if (wv == 0 && lane < TH) {
        lb0 = a.lb[bi];
        ub0 = a.ub[bi];
    }

    Vec<VEC> dl[RPT], du[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (i * RG < a.D) {
            if (NTL) {
                dl[i].load_nt(p_lw + i * row_step);
                du[i].load_nt(p_uw + i * row_step);
            } else {
                dl[i].load(p_lw + i * row_step);
                du[i].load(p_uw + i * row_step);
            }
        } else {
            dl[i].zero();
            du[i].zero();
        }
    }
    resident_partials<Q, VEC, RPT, RG, TPR, NW, TH>(a, dl, du, part, rg, c, lane, wv);
    __syncthreads();

    neuron_stage<MODE, Q, NW, TH>(a, part, s_lu, s_ln, lb0, ub0, a.l, a.u, bi, lane < TH, lane, wv);
    if (MODE == CONCRETIZE) return;

    float klo[VEC], kup[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        klo[v] = s_ln[c * VEC + v];
        kup[v] = s_ln[3 * TH + c * VEC + v];
    }
    float *__restrict__ q_lw = a.olw + base, *__restrict__ q_uw = a.ouw + base;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (i * RG < a.D) {
            Vec<VEC> ol, ou;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
                const float xl = dl[i].get(v), xu = du[i].get(v);
                ol.set(v, (klo[v] > 0.f ? xl : xu) * klo[v]);
                ou.set(v, (kup[v] > 0.f ? xu : xl) * kup[v]);
            }
            ol.store(q_lw + i * row_step);
            ou.store(q_uw + i * row_step);
        }
    }
}

// The same tile on a persistent workgroup: the grid is sized to the machine, a workgroup walks tiles
// blockIdx.x, blockIdx.x + gridDim.x, ... and holds TWO tiles in registers -- the loads of the next tile are issued
// before the norms, the per-neuron stage and the stores of the current one.  The first round of one-tile workgroups
// all load, then all compute, then all store, and memory sits idle at every change of phase (it shows when nothing
// is cached: the phases are then memory latencies apart); here reads and writes are in flight together from the
// second tile on, as in a copy.  Arithmetic per tile is that of act_resident, bit for bit.
// The tile's LDS (partial norms, intervals, lines) is reused from tile to tile: whoever writes `part` for the next
// tile has read its slopes of this one, and the per-neuron stage writes lines only after the barrier that follows
// those writes.
template <int MODE, int Q, int TPR, int NTHREADS, int RPT, int WPE>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(WPE))) act_pipelined(const ActArgs a, const int n_tiles) {
    static_assert(MODE != CONCRETIZE, "a read-only pass has no phases to overlap");
    constexpr int VEC = 4, TH = TPR * VEC, RG = NTHREADS / TPR, NW = NTHREADS / WAVE;
    static_assert(TH <= WAVE && NW >= 4, "per-neuron stages use one lane per neuron in wavefronts 0 ... 3");
    extern __shared__ float smem[];
    float *part = smem;                           // [words][NW][2][TH] per-wavefront partial norms
    float *s_lu = part + a.words * NW * 2 * TH;   // [2][TH] concrete interval
    float *s_ln = s_lu + 2 * TH;                  // [2][3][TH] lower / upper line (k, x0, y0)

    const int tiles = a.H / TH;
    const int tid = threadIdx.x, lane = tid % WAVE, wv = tid / WAVE;
    const int c = tid % TPR, rg = tid / TPR;
    const size_t row_step = (size_t)RG * a.H;

    struct Tile {
        Vec<VEC> dl[RPT], du[RPT];
        float lb0, ub0;
    };
    auto base_of = [&](int t) { return ((size_t)(t / tiles) * a.D + rg) * a.H + (t % tiles) * TH + c * VEC; };
    auto bias_of = [&](int t) { return (size_t)(t / tiles) * a.H + (t % tiles) * TH + lane; };
    auto fetch = [&](int t, Tile &x) __attribute__((always_inline)) {
        x.lb0 = x.ub0 = 0.f;
        if (wv == 0 && lane < TH) {
            x.lb0 = a.lb[bias_of(t)];
            x.ub0 = a.ub[bias_of(t)];
        }
        const float *__restrict__ p_lw = a.lw + base_of(t), *__restrict__ p_uw = a.uw + base_of(t);
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            if (i * RG < a.D) {
                x.dl[i].load(p_lw + i * row_step);
                x.du[i].load(p_uw + i * row_step);
            } else {
                x.dl[i].zero();
                x.du[i].zero();
            }
        }
    };
    auto finish = [&](int t, Tile &x) __attribute__((always_inline)) {
        resident_partials<Q, VEC, RPT, RG, TPR, NW, TH>(a, x.dl, x.du, part, rg, c, lane, wv);
        __syncthreads();
        neuron_stage<MODE, Q, NW, TH>(a, part, s_lu, s_ln, x.lb0, x.ub0, a.l, a.u, bias_of(t), lane < TH, lane, wv);
        float klo[VEC], kup[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
            klo[v] = s_ln[c * VEC + v];
            kup[v] = s_ln[3 * TH + c * VEC + v];
        }
        float *__restrict__ q_lw = a.olw + base_of(t), *__restrict__ q_uw = a.ouw + base_of(t);
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            if (i * RG < a.D) {
                Vec<VEC> ol, ou;
#pragma unroll
                for (int v = 0; v < VEC; ++v) {
                    const float xl = x.dl[i].get(v), xu = x.du[i].get(v);
                    ol.set(v, (klo[v] > 0.f ? xl : xu) * klo[v]);
                    ou.set(v, (kup[v] > 0.f ? xu : xl) * kup[v]);
                }
                ol.store(q_lw + i * row_step);
                ou.store(q_uw + i * row_step);
            }
        }
    };

    // virtual tile v (workgroup w walks v = w, w + grid, ...) -> tile: with a.remap, XCD x (v % 8 == x) owns groups of
    // consecutive rows
    auto tile_of = [&](int v) {
        if (a.remap == 1) return (v % 8) * (n_tiles / 8) + v / 8;
        if (a.remap == 2) {
            const int idx = v / 8, x = v % 8;
            return (idx / tiles * 8 + x) * tiles + idx % tiles;
        }
        return v;
    };
    Tile A, B;
    int v = blockIdx.x;
    if (v >= n_tiles) return;
    fetch(tile_of(v), A);
    while (true) {
        int vn = v + gridDim.x;
        if (vn < n_tiles) fetch(tile_of(vn), B);
        finish(tile_of(v), A);
        if (vn >= n_tiles) break;
        v = vn;
        vn = v + gridDim.x;
        if (vn < n_tiles) fetch(tile_of(vn), A);
        finish(tile_of(v), B);
        if (vn >= n_tiles) break;
        v = vn;
    }
}

// All modes, one neuron per lane (used by the transposed-layout kernel).
template <int MODE>
__device__ __forceinline__ void relax_any(float l, float u, float lb, float ub, float &klo, float &kup, float &olb,
                                          float &oub) {
    if (MODE == TANH) {
        Line lo, up;
        if (u < 0.f || l > 0.f) {
            tanh_pure_lines(l, u, lo, up);
        } else {
            lo = tanh_tangent_line<true>(l, u, tanh_tangent_point<true>(l, u), tanh_at(u).th);
            up = tanh_tangent_line<false>(l, u, tanh_tangent_point<false>(l, u), tanh_at(l).th);
        }
        klo = lo.k;
        kup = up.k;
        olb = line_bias(lo, lb, ub);
        oub = line_bias(up, ub, lb);
    } else {
        relax_point<MODE>(l, u, lb, ub, klo, kup, olb, oub);
    }
}

// ------------------------------------------------------------------ transposed layout
// Butterfly over the 64 lanes, every lane ends with the total.  Distances 1 to 8 are lane permutations inside a
// row of 16 lanes, done by the vector ALU on its own operand (DPP) instead of a trip through the LDS crossbar: 1 and
// 2 as permutations of four lanes; after them the four lanes of a group hold one value, so mirroring eight lanes
// fetches what lane ^ 4 holds, and after that mirroring sixteen fetches what lane ^ 8 holds.  16 and 32 go through
// the crossbar.
__device__ __forceinline__ float wave_sum(float v) {
    v += lane_permute<0xB1>(v);       // lanes 1 0 3 2
    v += lane_permute<0x4E>(v);       // lanes 2 3 0 1
    v += lane_permute<0x141>(v);      // eight lanes mirrored
    v += lane_permute<0x140>(v);      // sixteen lanes mirrored
    v += __shfl_xor(v, 16, WAVE);
    v += __shfl_xor(v, 32, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, lane_permute<0xB1>(v));
    v = fmaxf(v, lane_permute<0x4E>(v));
    v = fmaxf(v, lane_permute<0x141>(v));
    v = fmaxf(v, lane_permute<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    v = fmaxf(v, __shfl_xor(v, 32, WAVE));
    return v;
}
// 256 threads, 64 neurons per workgroup: each wavefront reduces 16 neurons (lanes along D_in,
// cross-lane butterfly), wavefront 0 then derives the 64 pairs of lines (one neuron per lane),
// and each wavefront scales its 16 neurons (second read comes from L2).
template <int MODE, int Q>
__global__ void __launch_bounds__(256) act_transposed(const ActArgs a) {
    constexpr int NPB = 64, NPW = NPB / 4;
    __shared__ float s_l[NPB], s_u[NPB], s_klo[NPB], s_kup[NPB];
    const long long total = (long long)a.rows * a.H;
    const long long n0 = (long long)blockIdx.x * NPB;
    const int lane = threadIdx.x % WAVE, wv = threadIdx.x / WAVE;
    const int blk = a.D / a.words;

    for (int i = 0; i < NPW; ++i) {
        const int t = wv * NPW + i;
        const long long n = n0 + t;
        if (n >= total) break;
        const float *pl = a.lw + (size_t)n * a.D, *pu = a.uw + (size_t)n * a.D;
        float l = a.lb[n], u = a.ub[n];
        for (int w = 0; w < a.words; ++w) {
            float nl = 0.f, nu = 0.f;
            for (int k = w * blk + lane; k < (w + 1) * blk; k += WAVE) {
                nl = nacc<Q>(nl, pl[k], a.qv);
                nu = nacc<Q>(nu, pu[k], a.qv);
            }
            nl = Q == FAITH_Q_INF ? wave_max(nl) : wave_sum(nl);
            nu = Q == FAITH_Q_INF ? wave_max(nu) : wave_sum(nu);
            l += (-a.eps) * nfin<Q>(nl, a.qv);
            u += a.eps * nfin<Q>(nu, a.qv);
        }
        if (lane == 0) {
            s_l[t] = l;
            s_u[t] = u;
            if (a.l) a.l[n] = l;
            if (a.u) a.u[n] = u;
        }
    }
    if (MODE == CONCRETIZE) return;
    __syncthreads();
    if (threadIdx.x < NPB && n0 + threadIdx.x < total) {
        const long long n = n0 + threadIdx.x;
        float klo, kup, olb, oub;
        relax_any<MODE>(s_l[threadIdx.x], s_u[threadIdx.x], a.lb[n], a.ub[n], klo, kup, olb, oub);
        s_klo[threadIdx.x] = klo;
        s_kup[threadIdx.x] = kup;
        a.olb[n] = olb;
        a.oub[n] = oub;
    }
    __syncthreads();
    for (int i = 0; i < NPW; ++i) {
        const int t = wv * NPW + i;
        const long long n = n0 + t;
        if (n >= total) break;
        const float klo = s_klo[t], kup = s_kup[t];
        const size_t off = (size_t)n * a.D;
        for (int k = lane; k < a.D; k += WAVE) {
            const float xl = a.lw[off + k], xu = a.uw[off + k];
            a.olw[off + k] = (klo > 0.f ? xl : xu) * klo;
            a.ouw[off + k] = (kup > 0.f ? xu : xl) * kup;
        }
    }
}

// ------------------------------------------------------------------ host dispatch
template <int MODE, int Q, int VEC, int TPR, int NTHREADS, int RPT>
void launch_natural(const ActArgs &a0, hipStream_t st) {
    constexpr int TH = TPR * VEC;
    ActArgs a = a0;
    const int tiles = (a.H + TH - 1) / TH;
    const size_t smem = ((size_t)a.words * (NTHREADS / WAVE) * 2 * TH + 8 * TH) * sizeof(float);
    const int tiles2 = (a.H2 + TH - 1) / TH;
    // the XCD-aware tile order of the register-resident kernels (dispatch_natural), where the row counts allow it
    const int tv = faith::tune_get(FAITH_TUNE_ACT_VARIANT);
    a.remap = (tv == 0 && a.rows % 8 == 0 && tiles > 1 && (a.rows2 == 0 || (a.rows2 % 8 == 0 && ((long long)a.rows * tiles) % 8 == 0))) ? 2 : 0;
    // rows that do not start on 64-byte boundaries ([128, 256, 300]: 45 -> 30 us, [128, 768, 300]: 173 -> 142 us)
    a.cached_stores = a.H % 16 != 0 ? 1 : 0;
    faith::reserve_lds(act_natural<MODE, Q, VEC, TPR, NTHREADS, RPT>, smem);      // many perturbed words: beyond 64 KB
    hipLaunchKernelGGL((act_natural<MODE, Q, VEC, TPR, NTHREADS, RPT>), dim3((unsigned)(a.rows * tiles + a.rows2 * tiles2)),
                       dim3(NTHREADS), smem, st, a);
}

template <int MODE, int Q, int TPR, int NTHREADS, int RPT, int WPE = 4, bool NTL = false, int MAXW = 8>
void launch_resident(const ActArgs &a, hipStream_t st) {
    constexpr int TH = TPR * 4;
    const size_t smem = ((size_t)a.words * (NTHREADS / WAVE) * 2 * TH + 8 * TH) * sizeof(float);
    faith::reserve_lds(act_resident<MODE, Q, TPR, NTHREADS, RPT, WPE, NTL, MAXW>, smem);
    hipLaunchKernelGGL((act_resident<MODE, Q, TPR, NTHREADS, RPT, WPE, NTL, MAXW>), dim3((unsigned)(a.rows * (a.H / TH))), dim3(NTHREADS),
                       smem, st, a);
}

template <int MODE, int Q, int TPR, int NTHREADS, int RPT, int WPE>
void launch_pipelined(const ActArgs &a, hipStream_t st) {
    constexpr int TH = TPR * 4;
    const size_t smem = ((size_t)a.words * (NTHREADS / WAVE) * 2 * TH + 8 * TH) * sizeof(float);
    faith::reserve_lds(act_pipelined<MODE, Q, TPR, NTHREADS, RPT, WPE>, smem);
    const int n_tiles = a.rows * (a.H / TH);
    // as many workgroups as are resident at once (WPE wavefronts per SIMD), no more than there are tiles
    const int resident = faith::compute_units() * (4 * WPE / (NTHREADS / WAVE));
    hipLaunchKernelGGL((act_pipelined<MODE, Q, TPR, NTHREADS, RPT, WPE>), dim3((unsigned)std::min(n_tiles, resident)), dim3(NTHREADS),
                       smem, st, a, n_tiles);
}

// Butterflies over groups of F lanes (F = 8, 16, 32 side by side in a wavefront), every lane ends with its group's
// total: the steps of wave_sum / wave_max up to distance F / 2.
template <int F>
__device__ __forceinline__ float group_sum(float v) {
    v += lane_permute<0xB1>(v);
    v += lane_permute<0x4E>(v);
    v += lane_permute<0x141>(v);
    if constexpr (F >= 16) v += lane_permute<0x140>(v);
    if constexpr (F >= 32) v += __shfl_xor(v, 16, WAVE);
    if constexpr (F >= 64) v += __shfl_xor(v, 32, WAVE);
    return v;
}
template <int F>
__device__ __forceinline__ float group_max(float v) {
    v = fmaxf(v, lane_permute<0xB1>(v));
    v = fmaxf(v, lane_permute<0x4E>(v));
    v = fmaxf(v, lane_permute<0x141>(v));
    if constexpr (F >= 16) v = fmaxf(v, lane_permute<0x140>(v));
    if constexpr (F >= 32) v = fmaxf(v, __shfl_xor(v, 16, WAVE));
    if constexpr (F >= 64) v = fmaxf(v, __shfl_xor(v, 32, WAVE));
    return v;
}

// Transposed layout, D_in a multiple of 4 up to 1024, 16-byte aligned: a neuron's D_in coefficients are one
// contiguous row, which the lanes of a wavefront read 16 bytes each -- V loads per lane for rows of more than 256
// floats (V = ceil(D_in / 256); lanes past the end of the row hold zeros), G = 64 / (D_in / 4) neurons side by side
// for rows of 128, 64 or 32 floats.  A wavefront owns R G neurons, and everything it reads (up to 64 values per
// thread) stays in registers between the norm and the scaling: one read, one write, no LDS and no barrier.  The
// norms of a neuron end up in every lane of its group (butterfly); lane j then derives the lines of the
// wavefront's j-th neuron, and the slopes travel back by cross-lane reads.
template <int MODE, int Q, int V, int G, int R>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) act_transposed_resident(const ActArgs a) {
    static_assert(V == 1 || G == 1, "several loads per lane, or several neurons per row of lanes");
    constexpr int NPW = R * G, F = WAVE / G;                           // neurons per wavefront; lanes per neuron
    static_assert(4 * NPW <= WAVE, "the shared tanh stage takes one neuron per lane of a wavefront");
    const int lane = threadIdx.x % WAVE, wv = threadIdx.x / WAVE;
    const int grp = G == 1 ? 0 : lane / F, fl = G == 1 ? lane : lane % F;
    const long long total = (long long)a.rows * a.H;
    const long long n0 = ((long long)blockIdx.x * 4 + wv) * NPW;      // first neuron of this wavefront
    const int blk = a.D / a.words;
    bool ok[V];
#pragma unroll
    for (int v = 0; v < V; ++v) ok[v] = (v * WAVE + fl) * 4 < a.D;

    Vec<4> dl[R][V], du[R][V];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const long long want = n0 + i * G + grp;
        const long long n = want < total ? want : total - 1;          // a clamped neuron is never stored
        const float *pl = a.lw + (size_t)n * a.D + fl * 4, *pu = a.uw + (size_t)n * a.D + fl * 4;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            if (ok[v]) {
                dl[i][v].load(pl + v * 256);
                du[i][v].load(pu + v * 256);
            } else {
                dl[i][v].zero();
                du[i][v].zero();
            }
        }
    }
    float l[R], u[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const long long want = n0 + i * G + grp;
        const long long n = want < total ? want : total - 1;
        float li = a.lb[n], ui = a.ub[n];
        for (int w = 0; w < a.words; ++w) {
            float nl = 0.f, nu = 0.f;
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const int k0 = (v * WAVE + fl) * 4;                   // blk % 4 == 0: a float4 lies in one word
                if (k0 >= w * blk && k0 < (w + 1) * blk) {            // (zeros past the end of the row belong to none)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        nl = nacc<Q>(nl, dl[i][v].get(c), a.qv);
                        nu = nacc<Q>(nu, du[i][v].get(c), a.qv);
                    }
                }
            }
            nl = Q == FAITH_Q_INF ? group_max<F>(nl) : group_sum<F>(nl);
            nu = Q == FAITH_Q_INF ? group_max<F>(nu) : group_sum<F>(nu);
            li += (-a.eps) * nfin<Q>(nl, a.qv);
            ui += a.eps * nfin<Q>(nu, a.qv);
        }
        l[i] = li;
        u[i] = ui;
    }
    // lane j takes the wavefront's j-th neuron: row j / G of group j % G
    float myl = 0.f, myu = 0.f;
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const float tl = G == 1 ? l[i] : __shfl(l[i], (lane % G) * F, WAVE);
        const float tu = G == 1 ? u[i] : __shfl(u[i], (lane % G) * F, WAVE);
        if (lane / G == i) {
            myl = tl;
            myu = tu;
        }
    }
    float klo = 0.f, kup = 0.f;
    const long long mine = n0 + lane;
    if (lane < NPW && mine < total) {
        if (a.l) a.l[mine] = myl;
        if (a.u) a.u[mine] = myu;
        if (MODE != CONCRETIZE && MODE != TANH) {
            float olb, oub;
            relax_any<MODE>(myl, myu, a.lb[mine], a.ub[mine], klo, kup, olb, oub);
            a.olb[mine] = olb;
            a.oub[mine] = oub;
        }
    }
    if (MODE == CONCRETIZE) return;
    if (MODE == TANH) {
        // the search for the tangent points is long: gather the workgroup's neurons in LDS and let four
        // wavefronts do it for all of them at once, one neuron per lane
        constexpr int NPB = 4 * NPW;
        __shared__ float s_lu[2 * NPB], s_ln[6 * NPB];
        if (lane < NPW) {
            s_lu[wv * NPW + lane] = myl;
            s_lu[NPB + wv * NPW + lane] = myu;
        }
        __syncthreads();
        const long long first = (long long)blockIdx.x * NPB;
        const bool mine_ok = lane < NPB && first + lane < total;
        const float lb0 = (wv == 0 && mine_ok) ? a.lb[first + lane] : 0.f, ub0 = (wv == 0 && mine_ok) ? a.ub[first + lane] : 0.f;
        tanh_stage<NPB>(a, s_lu, s_ln, lb0, ub0, (size_t)(first + lane), mine_ok, lane, wv);
        if (lane < NPW) {
            klo = s_ln[wv * NPW + lane];
            kup = s_ln[3 * NPB + wv * NPW + lane];
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const float k_lo = __shfl(klo, i * G + grp, WAVE), k_up = __shfl(kup, i * G + grp, WAVE);
        const long long n = n0 + i * G + grp;
        if (n < total) {
            float *ql = a.olw + (size_t)n * a.D + fl * 4, *qu = a.ouw + (size_t)n * a.D + fl * 4;
#pragma unroll
            for (int v = 0; v < V; ++v) {
                if (ok[v]) {
                    Vec<4> ol, ou;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float xl = dl[i][v].get(c), xu = du[i][v].get(c);
                        ol.set(c, (k_lo > 0.f ? xl : xu) * k_lo);
                        ou.set(c, (k_up > 0.f ? xu : xl) * k_up);
                    }
                    ol.store(ql + v * 256);
                    ou.store(qu + v * 256);
                }
            }
        }
    }
}

template <int MODE, int Q>
void dispatch_natural(const ActArgs &a, hipStream_t st) {
    const bool vec4 = (a.H % 4 == 0) && (a.H2 % 4 == 0) && faith::aligned(a.lw, 16) && faith::aligned(a.uw, 16) &&
                      faith::aligned(a.lw2, 16) && faith::aligned(a.uw2, 16) &&
                      (MODE == CONCRETIZE || (faith::aligned(a.olw, 16) && faith::aligned(a.ouw, 16)));
    if (MODE == CONCRETIZE) {
        // nothing is kept, so what counts is bytes in flight: 64-neuron tiles, 16 wavefronts, 256 rows
        // per pass measured best or equal on every shape tried (wide and narrow H alike) -- except
        // where a row of neurons is 64 KB or more (image-shaped bounds: every row of a tile then lies
        // on another page), where four-wavefront workgroups are 12 % ahead (6.2 against 5.4 TB/s at
        // configuration 4)
        if (!vec4 && a.rows2 > 0) {
            // two objects of which at least one cannot be read 16 bytes at a time (a row of attention
            // probabilities is as long as the sentence): a launch each, so that the other keeps its fast path
            ActArgs first = a, second = a;
            first.rows2 = 0;  first.H2 = 0;
            first.lb2 = first.ub2 = first.lw2 = first.uw2 = nullptr;  first.l2 = first.u2 = nullptr;
            second.lb = a.lb2;  second.ub = a.ub2;  second.lw = a.lw2;  second.uw = a.uw2;
            second.l = a.l2;  second.u = a.u2;  second.rows = a.rows2;  second.H = a.H2;
            second.rows2 = 0;  second.H2 = 0;
            second.lb2 = second.ub2 = second.lw2 = second.uw2 = nullptr;  second.l2 = second.u2 = nullptr;
            dispatch_natural<MODE, Q>(first, st);
            dispatch_natural<MODE, Q>(second, st);
            return;
        }
        const int pick = faith::tune_get(FAITH_TUNE_ACT_VARIANT);
        // ... and where the objects are large (64 MB and more: the operands of a configuration-size dot product),
        // where many small workgroups that start and finish at different times keep the memory system busier
        // than two rounds of sixteen-wavefront ones: 23.8 against 25.4 us at 134 MB, 23.2 against 25.7 us at
        // [512, 256, 128]
        const long long bytes = 8LL * a.D * ((long long)a.rows * a.H + (long long)a.rows2 * a.H2);
        if (vec4 && (pick == 11 || (pick == 0 && ((long long)a.H * 4 >= 65536 || bytes >= (64LL << 20)))))
            launch_natural<MODE, Q, 4, 16, 256, 8>(a, st);
        else if (vec4 && pick == 13)
            launch_natural<MODE, Q, 4, 8, 256, 8>(a, st);
        else if (vec4)
            launch_natural<MODE, Q, 4, 16, 1024, 4>(a, st);
        else if (a.H <= 8 && a.H2 <= 8)
            // a handful of neurons (the margin of a classifier): 64-neuron tiles would walk D_in in chunks of
            // 32 rows, one memory latency each; 8-neuron tiles take 256 rows per chunk
            launch_natural<MODE, Q, 1, 8, 256, 8>(a, st);
        else if (a.H <= 32 && a.H2 <= 32)
            launch_natural<MODE, Q, 1, 32, 256, 8>(a, st);      // no lane without a neuron, 64 rows per chunk
        else
            launch_natural<MODE, Q, 1, 64, 256, 8>(a, st);
        return;
    }
    if (!vec4) {
        launch_natural<MODE, Q, 1, 64, 256, 16>(a, st);   // 64 neurons x 64 rows per chunk
        return;
    }
    // straight-line kernel for the common shape: 32-neuron tiles, 32 rows in flight, up to 8 rows a thread
    const int tv = faith::tune_get(FAITH_TUNE_ACT_VARIANT);
    // 256 < D_in <= 1024 in whole steps of the tile (64 rows with eight wavefronts, 128 with sixteen; eight rows a
    // thread): the same straight-line kernel, where the general one below walks its tile with row and column
    // predicates -- same bits, [128, 512, 512] 110 -> 86 us, [32, 768, 768] 75 -> 50 us, [128, 1024, 512] 224 -> 203 us
    // (knob 9 keeps the general kernel)
    if constexpr (MODE != CONCRETIZE && Q != Q_GENERAL) {
        if (tv == 0 && a.rows2 == 0 && a.H % 32 == 0 && a.D > 256 && a.D <= 1024) {
            ActArgs b = a;
            b.remap = a.rows % 8 == 0 ? 2 : 0;
            if (a.D <= 512 && a.D % 64 == 0) { launch_resident<MODE, Q, 8, 512, 8, 4, false, 4>(b, st); return; }
            if (a.D % 128 == 0) { launch_resident<MODE, Q, 8, 1024, 8, 4, false, 4>(b, st); return; }
        }
    }
    if (tv != 9 && a.rows2 == 0 && a.H % 32 == 0 && a.D % 32 == 0 && a.D <= 256) {
        // Tile order (ActArgs::remap): the hardware deals consecutive workgroups to the eight XCDs in turn, so with
        // tiles numbered along a row every XCD touches every row of the object at once; with whole rows dealt to the
        // XCDs (row r to XCD r % 8) the workgroups of an XCD stream through consecutive tiles.  Four wavefronts x 8
        // rows on [128, 256, 512], relu / tanh: 61 / 64 -> 56 / 59 us when every byte comes from and goes to HBM
        // ("cold": five operand sets in turn), 41 / 40 -> 40 / 40 us when every launch reuses one set, which can sit in
        // the 256 MB memory-side cache ("warm").  Needs rows % 8 == 0 (else: an eighth of the tile range per XCD when
        // the tile count allows, else the plain order).
        // How many tiles a CU has in flight decides between the two regimes (same object, XCD-aware order, warm | cold, us):
        //   4 wavefronts x 8 rows, 4 workgroups per CU (256 KB in flight)   relu 39.9 | 56.0   tanh 40.5 | 59.3
        //   4 wavefronts x 8 rows, 3 per CU                                 relu 40.9 | 53.9   tanh 42.1 | 55.0
        //   4 wavefronts x 8 rows, 2 per CU                                 relu 42.9 | 52.7   tanh 45.2 | 56.6
        //   8 wavefronts x 4 rows, 3 per CU (192 KB)                        relu 40.8 | 53.8   tanh 40.7 | 54.4
        //   8 wavefronts x 4 rows, 2 per CU (128 KB)                        relu 41.4 | 51.9   tanh 42.7 | 52.7
        //   16 wavefronts x 2 rows, 2 per CU                                relu 44.5 | 52.7   tanh 48.0 | 53.6
        //   the same with non-temporal loads                                relu 50.2 | 51.3   tanh 51.3 | 52.5
        //   persistent, two tiles in registers, 2 per CU (plain order)      relu 41.5 | 57.3   tanh 43.8 | 59.9
        //   the same with whole rows per XCD, 4 / 8 wavefronts              relu 41.8 | 58.2, 42.3 | 59.4   tanh 42.1 | 60.6, 43.2 | 62.4
        // From the cache more tiles in flight are better, from HBM fewer; the library cannot know which it will be, so
        // the default is the shape that is within 4 % of the best in both: eight wavefronts, two workgroups per CU --
        // three for tanh, whose per-neuron stage (ten dependent bisection steps on two of the wavefronts) wants a
        // third workgroup to run meanwhile.  Objects whose traffic is beyond 9/4 of the cache cannot be resident in it:
        // sixteen wavefronts and non-temporal loads ([B, 32, 256, 512], 404 MB ... 2 GB: the order flips near 600 MB).
        // Knob values 8 / 12 / 7 force the one-tile shapes of four / sixteen / sixteen wavefronts with non-temporal loads
        // in the plain tile order, 15 the persistent kernel.
        const long long traffic = 16LL * a.rows * a.D * a.H;
        const bool streams_from_hbm = tv == 7 || (tv != 8 && traffic > 9LL * (256LL << 20) / 4);
        if constexpr (MODE != CONCRETIZE) {
            if (a.D > 128 && tv == 15) {
                launch_pipelined<MODE, Q, 8, 256, 8, 2>(a, st);
                return;
            }
        }
        ActArgs b = a;
        const long long n_tiles = (long long)a.rows * (a.H / 32);
        b.remap = (tv == 8 || tv == 12 || tv == 7) ? 0 : a.rows % 8 == 0 ? 2 : n_tiles % 8 == 0 ? 1 : 0;
        // a step of the tile is NTHREADS / 8 rows, whole steps only: the shapes of eight and sixteen wavefronts take
        // D_in that are multiples of 64 and of 128; 160 or 224 rows stay with four wavefronts (steps of 32 rows)
        const bool steps64 = a.D % 64 == 0, steps128 = a.D % 128 == 0;
        if (a.D <= 128) launch_resident<MODE, Q, 8, 256, 4>(b, st);
        else if (tv == 12 && steps128) launch_resident<MODE, Q, 8, 1024, 2, 8, false>(b, st);
        else if (streams_from_hbm && steps128) launch_resident<MODE, Q, 8, 1024, 2, 8, true>(b, st);
        else if (tv == 8 || Q == Q_GENERAL || MODE == CONCRETIZE || !steps64)
            launch_resident<MODE, Q, 8, 256, 8, (Q == Q_GENERAL ? 3 : 4)>(b, st);     // a general exponent needs more registers than 128
        else if (MODE == TANH) launch_resident<MODE, Q, 8, 512, 4, 6, false, 6>(b, st);
        else launch_resident<MODE, Q, 8, 512, 4, 4, false, 4>(b, st);
        return;
    }
    switch (tv) {
        case 1: launch_natural<MODE, Q, 4, 8, 256, 8>(a, st); return;     // 32 neurons, 256 rows / chunk
        case 2: launch_natural<MODE, Q, 4, 16, 512, 8>(a, st); return;    // 64 neurons, 256 rows / chunk, 8 waves
        case 3: launch_natural<MODE, Q, 4, 16, 1024, 4>(a, st); return;   // 64 neurons, 256 rows / chunk, 16 waves
        case 4: launch_natural<MODE, Q, 4, 8, 512, 4>(a, st); return;     // 32 neurons, 256 rows / chunk, 8 waves
        case 5: launch_natural<MODE, Q, 4, 16, 256, 16>(a, st); return;   // 64 neurons, 256 rows / chunk, 4 waves
        case 6: launch_natural<MODE, Q, 4, 8, 1024, 8>(a, st); return;    // 32 neurons, 1024 rows / chunk, 16 waves
        default: break;
    }
    // 32-neuron tiles (128-byte row segments) keep the register footprint at 64 values per
    // thread, which measured fastest on MI355X (more resident workgroups, shorter tail).
    if (a.D <= 128) {
        launch_natural<MODE, Q, 4, 8, 256, 4>(a, st);     // D_in <= 128 in registers
    } else if (a.D <= 256) {
        launch_natural<MODE, Q, 4, 8, 256, 8>(a, st);     // D_in <= 256 in registers
    } else if (a.D <= 512 || a.D > 1024) {
        launch_natural<MODE, Q, 4, 8, 512, 8>(a, st);     // D_in <= 512 in registers, chunks beyond
    } else {
        // D_in <= 1024 in the registers of sixteen wavefronts: one read instead of two (8 - 13 % ahead
        // of the chunked walk at D_in = 640 ... 1024)
        launch_natural<MODE, Q, 4, 8, 1024, 8>(a, st);
    }
}

template <int MODE, int Q>
void dispatch_layout(const ActArgs &a, int layout, hipStream_t st) {
    if (layout == FAITH_LAYOUT_NATURAL) {
        dispatch_natural<MODE, Q>(a, st);
    } else {
        const long long total = (long long)a.rows * a.H;
        const bool vec = (a.D / a.words) % 4 == 0 && faith::aligned(a.lw, 16) && faith::aligned(a.uw, 16) &&
                         (MODE == CONCRETIZE || (faith::aligned(a.olw, 16) && faith::aligned(a.ouw, 16)));
        // rows of up to 1024 floats stay in registers (see act_transposed_resident): V loads per lane, or G neurons
        // side by side in a wavefront
        auto resident = [&](auto v, auto g, auto r) {
            constexpr int V = decltype(v)::value, G = decltype(g)::value, R = decltype(r)::value;
            hipLaunchKernelGGL((act_transposed_resident<MODE, Q, V, G, R>), dim3((unsigned)((total + 4 * R * G - 1) / (4 * R * G))),
                               dim3(256), 0, st, a);
        };
        using std::integral_constant;
        const int f4 = a.D / 4;
        if (vec && a.D == 128) resident(integral_constant<int, 1>{}, integral_constant<int, 2>{}, integral_constant<int, 8>{});
        else if (vec && a.D == 64) resident(integral_constant<int, 1>{}, integral_constant<int, 4>{}, integral_constant<int, 4>{});
        else if (vec && a.D == 32) resident(integral_constant<int, 1>{}, integral_constant<int, 8>{}, integral_constant<int, 2>{});
        else if (vec && f4 <= 64) resident(integral_constant<int, 1>{}, integral_constant<int, 1>{}, integral_constant<int, 8>{});
        else if (vec && f4 <= 128) resident(integral_constant<int, 2>{}, integral_constant<int, 1>{}, integral_constant<int, 4>{});
        else if (vec && f4 <= 192) resident(integral_constant<int, 3>{}, integral_constant<int, 1>{}, integral_constant<int, 2>{});
        else if (vec && f4 <= 256) resident(integral_constant<int, 4>{}, integral_constant<int, 1>{}, integral_constant<int, 2>{});
        else
            hipLaunchKernelGGL((act_transposed<MODE, Q>), dim3((unsigned)((total + 63) / 64)), dim3(256), 0, st, a);
    }
}

template <int MODE>
int run(const char *who, ActArgs a, int q, int layout, void *stream) {
    FAITH_REQUIRE(a.rows > 0 && a.D > 0 && a.H > 0, FAITH_ERR_SHAPE,
                  "%s: rows=%d dim_in=%d dim_out=%d must all be positive", who, a.rows, a.D, a.H);
    FAITH_REQUIRE(a.words >= 1 && a.words <= 16 && a.D % a.words == 0, FAITH_ERR_SHAPE,
                  "%s: words=%d must be in 1..16 and divide dim_in=%d", who, a.words, a.D);
    if (!faith::dual_exponent(q, &a.qv)) {
        faith::set_error("%s: q=%d is neither FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF nor the bits of an exponent in (1, inf)", who, q);
        return FAITH_ERR_UNSUPPORTED;
    }
    FAITH_REQUIRE(layout == FAITH_LAYOUT_NATURAL || layout == FAITH_LAYOUT_TRANSPOSED, FAITH_ERR_UNSUPPORTED,
                  "%s: unknown layout %d", who, layout);
    FAITH_REQUIRE((long long)a.rows * a.H * 1LL <= 0x7fffffffLL * 32, FAITH_ERR_SHAPE, "%s: problem too large", who);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (q) {
        case FAITH_Q_1: dispatch_layout<MODE, FAITH_Q_1>(a, layout, st); break;
        case FAITH_Q_2: dispatch_layout<MODE, FAITH_Q_2>(a, layout, st); break;
        case FAITH_Q_INF: dispatch_layout<MODE, FAITH_Q_INF>(a, layout, st); break;
        default: dispatch_layout<MODE, Q_GENERAL>(a, layout, st); break;
    }
    return faith::check_launch(who);
}

// ------------------------------------------------------------------ concrete interval of a compact object
// An object that keeps the coefficient rows of P positions per batch element only (zero elsewhere: the input of a
// query, VerifierForward.py:127-156, and what layer norm and dense layers make of it): its interval is the constant
// terms everywhere and lb -/+ eps * ||rows|| (Bounds.py:311-326) at those positions.  One launch: the first `norm_wgs`
// workgroups take one (batch element, position, 64 neurons) each -- four wavefronts over the dim_in rows of every
// word's block, partial norms through LDS, the words added in the reference's order --, the others copy the
// constants of the positions that have no coefficients.  A position outside 0 .. L-1 names no row.
struct RowsArgs {
    const float *lb, *ub, *lw, *uw;       // [B, L, H]; [B, P, D, H]
    const long long *positions;           // [B, P]
    float *l, *u;                         // [B, L, H]
    int B, L, P, D, H, words;
    float eps, qv;
};
template <int Q>
__global__ void __launch_bounds__(256) concretize_rows_kernel(const RowsArgs a, const int norm_wgs) {
    __shared__ float part[16 * 4 * 2 * 64];                 // [word][row group][l, u][column]
    const int tid = threadIdx.x;
    if ((int)blockIdx.x >= norm_wgs) {
        // constants of the other positions, 4 bytes per thread and step
        const size_t n = (size_t)a.B * a.L * a.H, stride = (size_t)(gridDim.x - norm_wgs) * 256;
        for (size_t e = (size_t)(blockIdx.x - norm_wgs) * 256 + tid; e < n; e += stride) {
            const size_t bl = e / a.H;
            const size_t bb = bl / a.L;
            const long long l = (long long)(bl % a.L);
            bool mine = true;
            for (int p = 0; p < a.P; ++p) mine = mine && a.positions[bb * a.P + p] != l;
            if (mine) {
                a.l[e] = a.lb[e];
                a.u[e] = a.ub[e];
            }
        }
        return;
    }
    const int tiles = (a.H + 63) / 64;
    const int bp = blockIdx.x / tiles, col = (blockIdx.x % tiles) * 64 + tid % 64, rg = tid / 64;
    const long long at = a.positions[bp];
    if (at < 0 || at >= a.L) return;                        // uniform over the workgroup
    const bool col_ok = col < a.H;
    const int blk = a.D / a.words;
    const float *lw = a.lw + (size_t)bp * a.D * a.H + col, *uw = a.uw + (size_t)bp * a.D * a.H + col;
    for (int w = 0; w < a.words; ++w) {
        float nl = 0.f, nu = 0.f;
        if (col_ok) {
#pragma unroll 4
            for (int d = w * blk + rg; d < (w + 1) * blk; d += 4) {
                nl = nacc<Q>(nl, lw[(size_t)d * a.H], a.qv);
                nu = nacc<Q>(nu, uw[(size_t)d * a.H], a.qv);
            }
        }
        part[((w * 4 + rg) * 2 + 0) * 64 + tid % 64] = nl;
        part[((w * 4 + rg) * 2 + 1) * 64 + tid % 64] = nu;
    }
    __syncthreads();
    if (rg == 0 && col_ok) {
        const size_t o = ((size_t)(bp / a.P) * a.L + (size_t)at) * a.H + col;
        float l = a.lb[o], u = a.ub[o];
        for (int w = 0; w < a.words; ++w) {
            float nl = 0.f, nu = 0.f;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                nl = ncomb<Q>(nl, part[((w * 4 + g) * 2 + 0) * 64 + tid]);
                nu = ncomb<Q>(nu, part[((w * 4 + g) * 2 + 1) * 64 + tid]);
            }
            l += (-a.eps) * nfin<Q>(nl, a.qv);
            u += a.eps * nfin<Q>(nu, a.qv);
        }
        a.l[o] = l;
        a.u[o] = u;
    }
}

}  // namespace

extern "C" int faith_concretize_rows(const float *lb, const float *ub, const float *lw, const float *uw,
                                     const long long *positions, float *l, float *u, int batch_size, int length,
                                     int n_positions, int dim_in, int dim_out, float eps, int q, int words, void *stream) {
    const char *who = "faith_concretize_rows";
    FAITH_NOT_NULL(lb); FAITH_NOT_NULL(ub); FAITH_NOT_NULL(lw); FAITH_NOT_NULL(uw); FAITH_NOT_NULL(positions);
    FAITH_NOT_NULL(l); FAITH_NOT_NULL(u);
    FAITH_ALIGNED4(lb); FAITH_ALIGNED4(ub); FAITH_ALIGNED4(lw); FAITH_ALIGNED4(uw); FAITH_ALIGNED4(l); FAITH_ALIGNED4(u);
    FAITH_REQUIRE(faith::aligned(positions, 8), FAITH_ERR_ALIGN, "%s: positions is not 8-byte aligned", who);
    FAITH_REQUIRE(batch_size > 0 && length > 0 && n_positions > 0 && dim_in > 0 && dim_out > 0, FAITH_ERR_SHAPE,
                  "%s: batch=%d length=%d positions=%d dim_in=%d dim_out=%d must be positive", who, batch_size, length,
                  n_positions, dim_in, dim_out);
    FAITH_REQUIRE(words >= 1 && words <= 16 && dim_in % words == 0, FAITH_ERR_SHAPE,
                  "%s: words=%d must be in 1..16 and divide dim_in=%d", who, words, dim_in);
    RowsArgs a{lb, ub, lw, uw, positions, l, u, batch_size, length, n_positions, dim_in, dim_out, words, eps, 0.f};
    if (!faith::dual_exponent(q, &a.qv)) {
        faith::set_error("%s: q=%d is neither FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF nor the bits of an exponent in (1, inf)", who, q);
        return FAITH_ERR_UNSUPPORTED;
    }
    const long long norm_wgs = (long long)batch_size * n_positions * ((dim_out + 63) / 64);
    const long long elems = (long long)batch_size * length * dim_out;
    long long copy_wgs = (elems + 255) / 256;
    if (copy_wgs > 4096) copy_wgs = 4096;
    FAITH_REQUIRE(norm_wgs + copy_wgs <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
    const dim3 gd((unsigned)(norm_wgs + copy_wgs)), bd(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (q) {
        case FAITH_Q_1: hipLaunchKernelGGL(concretize_rows_kernel<FAITH_Q_1>, gd, bd, 0, st, a, (int)norm_wgs); break;
        case FAITH_Q_2: hipLaunchKernelGGL(concretize_rows_kernel<FAITH_Q_2>, gd, bd, 0, st, a, (int)norm_wgs); break;
        case FAITH_Q_INF: hipLaunchKernelGGL(concretize_rows_kernel<FAITH_Q_INF>, gd, bd, 0, st, a, (int)norm_wgs); break;
        default: hipLaunchKernelGGL(concretize_rows_kernel<Q_GENERAL>, gd, bd, 0, st, a, (int)norm_wgs); break;
    }
    return faith::check_launch(who);
}

// Concretizes two bound objects of equal dim_in in ONE launch (the dot product needs the intervals
// of both operands before it can start).  Natural layout.
int faith::concretize_pair(const float *lb, const float *ub, const float *lw, const float *uw, float *l, float *u,
                           int rows, const float *lb2, const float *ub2, const float *lw2, const float *uw2,
                           float *l2, float *u2, int rows2, int dim_in, int dim_out, int dim_out2, float eps, int q,
                           int words, void *stream, int layout) {
    ActArgs a{lb, ub, lw, uw, nullptr, nullptr, nullptr, nullptr, l, u, rows, dim_in, dim_out, words, eps};
    a.lb2 = lb2; a.ub2 = ub2; a.lw2 = lw2; a.uw2 = uw2; a.l2 = l2; a.u2 = u2; a.rows2 = rows2; a.H2 = dim_out2;
    return run<CONCRETIZE>("faith_concretize", a, q, layout, stream);
}

extern "C" int faith_concretize(const float *lb, const float *ub, const float *lw, const float *uw, float *l,
                                float *u, int rows, int dim_in, int dim_out, float eps, int q, int words,
                                int layout, void *stream) {
    FAITH_NOT_NULL(lb); FAITH_NOT_NULL(ub); FAITH_NOT_NULL(lw); FAITH_NOT_NULL(uw);
    FAITH_NOT_NULL(l); FAITH_NOT_NULL(u);
    FAITH_ALIGNED4(lb); FAITH_ALIGNED4(ub); FAITH_ALIGNED4(lw); FAITH_ALIGNED4(uw);
    FAITH_ALIGNED4(l); FAITH_ALIGNED4(u);
    ActArgs a{lb, ub, lw, uw, nullptr, nullptr, nullptr, nullptr, l, u, rows, dim_in, dim_out, words, eps};
    return run<CONCRETIZE>("faith_concretize", a, q, layout, stream);
}

static int act_entry(const char *who, int mode, const float *src_lb, const float *src_ub, const float *src_lw,
                     const float *src_uw, float *out_lb, float *out_ub, float *out_lw, float *out_uw,
                     float *l_out, float *u_out, int length, int dim_in, int dim_out, float epsilon, int q,
                     int words, int layout, void *stream) {
    FAITH_NOT_NULL(src_lb); FAITH_NOT_NULL(src_ub); FAITH_NOT_NULL(src_lw); FAITH_NOT_NULL(src_uw);
    FAITH_NOT_NULL(out_lb); FAITH_NOT_NULL(out_ub); FAITH_NOT_NULL(out_lw); FAITH_NOT_NULL(out_uw);
    FAITH_ALIGNED4(src_lb); FAITH_ALIGNED4(src_ub); FAITH_ALIGNED4(src_lw); FAITH_ALIGNED4(src_uw);
    FAITH_ALIGNED4(out_lb); FAITH_ALIGNED4(out_ub); FAITH_ALIGNED4(out_lw); FAITH_ALIGNED4(out_uw);
    FAITH_ALIGNED4(l_out); FAITH_ALIGNED4(u_out);
    ActArgs a{src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw, l_out, u_out,
              length, dim_in, dim_out, words, epsilon};
    switch (mode) {
        case RELU: return run<RELU>(who, a, q, layout, stream);
        case TANH: return run<TANH>(who, a, q, layout, stream);
        case EXP: return run<EXP>(who, a, q, layout, stream);
        case RECIP: return run<RECIP>(who, a, q, layout, stream);
        case SQR: return run<SQR>(who, a, q, layout, stream);
        case SQRT: return run<SQRT>(who, a, q, layout, stream);
        default:
            faith::set_error("%s: unknown relaxation %d", who, mode);
            return FAITH_ERR_UNSUPPORTED;
    }
}

extern "C" int faith_relu_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                       const float *src_uw, float *out_lb, float *out_ub, float *out_lw,
                                       float *out_uw, float *l_out, float *u_out, int length, int dim_in,
                                       int dim_out, float epsilon, int q, int words, int layout, void *stream) {
    return act_entry("faith_relu_verification", RELU, src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw,
                     out_uw, l_out, u_out, length, dim_in, dim_out, epsilon, q, words, layout, stream);
}

extern "C" int faith_tanh_verification(const float *src_lb, const float *src_ub, const float *src_lw,
                                       const float *src_uw, float *out_lb, float *out_ub, float *out_lw,
                                       float *out_uw, float *l_out, float *u_out, int length, int dim_in,
                                       int dim_out, float epsilon, int q, int words, int layout, void *stream) {
    return act_entry("faith_tanh_verification", TANH, src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw,
                     out_uw, l_out, u_out, length, dim_in, dim_out, epsilon, q, words, layout, stream);
}

extern "C" int faith_unary_verification(int op, const float *src_lb, const float *src_ub, const float *src_lw,
                                        const float *src_uw, float *out_lb, float *out_ub, float *out_lw,
                                        float *out_uw, float *l_out, float *u_out, int length, int dim_in,
                                        int dim_out, float epsilon, int q, int words, int layout, void *stream) {
    return act_entry("faith_unary_verification", op, src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw,
                     l_out, u_out, length, dim_in, dim_out, epsilon, q, words, layout, stream);
}

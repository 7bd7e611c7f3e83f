// The MFMA tile of the sign-split affine layer (the arithmetic, tiling and LDS layout are described at the top of
// gemm.hip).  A header because two translation units instantiate it: gemm.hip, with the macro-tiles the library
// ships, and variants/gemm_variant.hip, which faith_amd.autotune compiles with the tile shape and the scheduling
// switches below as macros -- the counterpart of the reference's autotuner rewriting matmul_config.h and
// recompiling (Transformer_Verification_Code/autotuner/).
//
//   FAITH_GEMM_SETPRIO   -1 (default): raised wavefront priority during a run of MFMAs for the 128 x 128 tile only;
//                        0 / 1: never / for every tile shape
#pragma once
#include "common.h"
#include "relax_lines.h"

#ifndef FAITH_GEMM_SETPRIO
#define FAITH_GEMM_SETPRIO -1
#endif

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int BK = 16;
constexpr int NTHREADS = 256;
constexpr int XCDS = 8;

struct GemmArgs {
    const float *Al, *Au;   // [Mw, K] coefficient rows (lower, upper)
    const float *Bl, *Bu;   // [Mb, K] constant-term rows
    const float *W;         // [N, K]
    const float *bias;      // [N] or nullptr
    float *Cl, *Cu;         // [Mw, N]
    float *Dl, *Du;         // [Mb, N]
    int Mw, Mb, N, K;
};

__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
// twice the centre, l + u, and twice the radius, u - l, of a pair of coefficients (the halving is left to the
// epilogue, where it is done once per result instead of once per operand element: it is exact either way); |w|
__device__ __forceinline__ float4 mid4(float4 l, float4 u) {
    return make_float4(l.x + u.x, l.y + u.y, l.z + u.z, l.w + u.w);
}
__device__ __forceinline__ float4 rad4(float4 l, float4 u) {
    return make_float4(u.x - l.x, u.y - l.y, u.z - l.z, u.w - l.w);
}
__device__ __forceinline__ float4 abs4(float4 v) {
    return make_float4(__builtin_fabsf(v.x), __builtin_fabsf(v.y), __builtin_fabsf(v.z), __builtin_fabsf(v.w));
}

// Accesses at or beyond `bytes` from the base are dropped by the hardware (loads return zero).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t window(const void *base, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0,
                                             (int)((bytes >> 32) ? 0xffffffffu : (unsigned)bytes), 0x00020000);
}
__device__ __forceinline__ float4 ld4(__amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(r, thread_off, uniform_off, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}

// position of 16-byte piece `c` (0 / 1) of row `row` inside a [128 x 8] half
__device__ __forceinline__ int swz(int row, int c) { return row * 8 + 4 * (c ^ ((row >> 2) & 1)); }

// EXACT = true: K % 16 == 0.  Otherwise (K % 4 == 0) the last K-step is partly past K: threads past
// it read their K-step-0 piece instead (in bounds) and discard it before it reaches LDS.
//
// MBM, MBN = MFMA blocks per wavefront along M and N: 2 x 2 is the 128 x 128 macro-tile described
// above; 1 x 1 is a 64 x 64 macro-tile (wavefront tile 32 x 32, 32 accumulator registers, 32 KB of LDS)
// for problems with too few 128 x 128 tiles to fill the machine: a wavefront then works through 32
// MFMAs per K-step instead of 128, a quarter of the latency, at a lower MFMA rate per byte staged.
// 2 x 1 and 1 x 2 (128 x 64, 64 x 128: 64 MFMAs per K-step, 48 KB) lie between.
// NQ >= 0 (a dual-norm selector): the tile's contribution to the column norms of C_l and C_u -- over its BM rows,
// which the caller guarantees to exist and to belong to one position -- is folded into pl / pu, one running
// value per lane and column block; NQ = -1: no norms.
// Epilogue of the tiles that hold whole rows of the result (the 64-row tile with all dim_y_out = 64 MBN columns):
// a second bound object is added and the rows go through the layer normalisation without the variance
// (Bounds.add, Bounds.layer_norm "no_var": Bounds.py:1016-1025, :1111-1131) before they are stored -- the sum
// and the layer's own result never reach memory.
struct RowNormArgs {
    const float *res_l, *res_u;     // coefficients of the added object, or null
    const long long *positions;     // null: its rows are the [Mw, N] rows of the result.  Otherwise it holds the dim_in
    int words, length, dim_in;      // rows of `words` positions per batch element only ([batch, words, dim_in, N];
                                    // positions [batch, words]): rows of other positions are zero
    const float *weight;            // [N] or null
    float *out_l, *out_u;           // [Mw, N]
};

// Epilogue of the tiles that hold every coefficient row of one position (BM = dim_in, one perturbed word): the
// column norms over those rows are complete inside the tile, so the concrete interval of each of its neurons and
// from it the two lines of the ReLU relaxation (Bounds.relu, Bounds.py:921-963) are known before the tile is
// stored -- the layer's own result never reaches memory.  The constant terms of the layer (g.Dl, g.Du) have been
// written by the launch before.
struct ReluArgs {
    float *out_lb, *out_ub;         // [Mb, N] constant terms behind the relaxation (may be g.Dl, g.Du themselves)
    float eps;
};

constexpr int EPI_PLAIN = 0, EPI_ROWNORM = 1, EPI_RELU = 2;

struct NoEpilogueArgs {};

template <bool EXACT, int MBM, int MBN, int NQ = -1, int EPI = EPI_PLAIN, class EpiArgs = NoEpilogueArgs>
__device__ __forceinline__ void signsplit_gemm_tile(const GemmArgs &g, float *smem, const int m_blk, const int n_blk,
                                                    float *pl = nullptr, float *pu = nullptr, float qv = 0.f,
                                                    const EpiArgs &epi = EpiArgs()) {
    constexpr int BM = 64 * MBM, BN = 64 * MBN;
    constexpr int HALF_A = BM * 8, HALF_W = BN * 8;      // floats in one [rows x 8] half of an operand's K-step
    constexpr int S_AM = 0, S_AR = 2 * HALF_A, S_W = 4 * HALF_A, S_WA = 4 * HALF_A + 2 * HALF_W;
    constexpr int STAGE = 4 * HALF_A + 4 * HALF_W;
    float(*sm)[STAGE] = reinterpret_cast<float(*)[STAGE]>(smem);

    const int M = g.Mw;
    const int m0 = m_blk * BM, n0 = n_blk * BN;
    const int K = g.K;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wm = wv / 2, wn = wv % 2;            // 2 x 2 wavefronts, (32 MBM) x (32 MBN) each

    // ---- staging: an operand's K-step is 64 or 128 rows x 16 floats, one float4 per thread and 64 rows:
    // piece kq of rows r0 (and r0 + 64).  Offsets are relative to the first row of the tile (the entry
    // point checks that a tile's rows span less than 4 GB); rows past the end re-read the last row, their
    // products are never stored.
    // (the two pieces of a row that belong to the K-step's second half are taken by the threads two rows away: the
    // eight lanes whose 16-byte stores the LDS serves in one cycle then write rows 0, 1 of the first half and rows
    // 2, 3 of the second -- eight different groups of banks -- instead of rows 0, 1 of both)
    const int kq = tid % 4, r0 = (tid / 4) ^ (kq & 2);
    const __amdgpu_buffer_rsrc_t wal = window(g.Al + (size_t)m0 * K, ((size_t)(M - m0) * K) * 4);
    const __amdgpu_buffer_rsrc_t wau = window(g.Au + (size_t)m0 * K, ((size_t)(M - m0) * K) * 4);
    const __amdgpu_buffer_rsrc_t ww = window(g.W + (size_t)n0 * K, ((size_t)(g.N - n0) * K) * 4);
    unsigned va[MBM], vw[MBN];
    int dsta[MBM], dstw[MBN];
#pragma unroll
    for (int i = 0; i < MBM; ++i) {
        const int ra = min(r0 + 64 * i, M - 1 - m0);
        va[i] = ((unsigned)ra * K + kq * 4) * 4u;
        dsta[i] = (kq / 2) * HALF_A + swz(r0 + 64 * i, kq % 2);
    }
#pragma unroll
    for (int i = 0; i < MBN; ++i) {
        const int rw = min(r0 + 64 * i, g.N - 1 - n0);
        vw[i] = ((unsigned)rw * K + kq * 4) * 4u;
        dstw[i] = (kq / 2) * HALF_W + swz(r0 + 64 * i, kq % 2);
    }
    const int nk = (K + BK - 1) / BK;
    float4 pal[MBM], pau[MBM], pw[MBN];
    auto past = [&](int kt) { return !EXACT && kt * BK + kq * 4 >= K; };
    auto gload = [&](int kt) {
        const unsigned k = kt * (BK * 4u);
        const unsigned kk = (!EXACT && past(kt)) ? 0u : k;     // !EXACT: the K offset travels with the thread
#pragma unroll
        for (int i = 0; i < MBM; ++i) {
            pal[i] = EXACT ? ld4(wal, va[i], k) : ld4(wal, va[i] + kk, 0);
            pau[i] = EXACT ? ld4(wau, va[i], k) : ld4(wau, va[i] + kk, 0);
        }
#pragma unroll
        for (int i = 0; i < MBN; ++i) pw[i] = EXACT ? ld4(ww, vw[i], k) : ld4(ww, vw[i] + kk, 0);
    };
    auto lstore = [&](int buf, int kt) {
        float *s = sm[buf];
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < MBM; ++i) {
            if (past(kt)) pal[i] = pau[i] = zero;
            *reinterpret_cast<float4 *>(s + S_AM + dsta[i]) = mid4(pal[i], pau[i]);
            *reinterpret_cast<float4 *>(s + S_AR + dsta[i]) = rad4(pal[i], pau[i]);
        }
#pragma unroll
        for (int i = 0; i < MBN; ++i) {
            if (past(kt)) pw[i] = zero;
            *reinterpret_cast<float4 *>(s + S_W + dstw[i]) = pw[i];
            *reinterpret_cast<float4 *>(s + S_WA + dstw[i]) = abs4(pw[i]);
        }
    };

    // cl accumulates twice the centre term, (A_l + A_u) . W, and cu twice the radius term, (A_u - A_l) . |W|; they become
    // C_l and C_u when the reduction is done
    floatx16 cl[MBM][MBN], cu[MBM][MBN];
#pragma unroll
    for (int a = 0; a < MBM; ++a)
#pragma unroll
        for (int b = 0; b < MBN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;

    // fragments: lane (fi = lane % 32, fh = lane / 32) reads k = 8*ks + 4*fh .. +3 of row fi
    const int fi = lane % 32, fh = lane / 32;
    int fa[MBM], fw[MBN];
#pragma unroll
    for (int s = 0; s < MBM; ++s) fa[s] = swz((wm * MBM + s) * 32 + fi, fh);
#pragma unroll
    for (int s = 0; s < MBN; ++s) fw[s] = swz((wn * MBN + s) * 32 + fi, fh);
    auto compute = [&](int buf, auto &&halfway) {
        const float *s = sm[buf];
#pragma unroll
        for (int ks = 0; ks < BK / 8; ++ks) {
            if (ks == 1) halfway();
            float4 am[MBM], ar[MBM], wp[MBN], wq[MBN];
#pragma unroll
            for (int t = 0; t < MBM; ++t) {
                am[t] = *reinterpret_cast<const float4 *>(s + S_AM + ks * HALF_A + fa[t]);
                ar[t] = *reinterpret_cast<const float4 *>(s + S_AR + ks * HALF_A + fa[t]);
            }
#pragma unroll
            for (int t = 0; t < MBN; ++t) {
                wp[t] = *reinterpret_cast<const float4 *>(s + S_W + ks * HALF_W + fw[t]);
                wq[t] = *reinterpret_cast<const float4 *>(s + S_WA + ks * HALF_W + fw[t]);
            }
#define FAITH_STEP(c)                                                           \
    _Pragma("unroll") for (int a = 0; a < MBM; ++a) _Pragma("unroll") for (int b = 0; b < MBN; ++b) { \
        cl[a][b] = mfma(am[a].c, wp[b].c, cl[a][b]);                            \
        cu[a][b] = mfma(ar[a].c, wq[b].c, cu[a][b]);                            \
    }
            // 128 x 128 only: a wavefront inside its run of 64 MFMAs goes before its neighbour's staging and
            // address arithmetic (configuration 2: 1.5 % faster; the small tiles, whose runs are 16 or 32
            // MFMAs between more frequent barriers, measured 1.5 % slower with it)
            constexpr bool PRIO = FAITH_GEMM_SETPRIO < 0 ? (MBM == 2 && MBN == 2) : FAITH_GEMM_SETPRIO != 0;
            if (PRIO) __builtin_amdgcn_s_setprio(1);
            FAITH_STEP(x)
            FAITH_STEP(y)
            FAITH_STEP(z)
            FAITH_STEP(w)
            if (PRIO) __builtin_amdgcn_s_setprio(0);
#undef FAITH_STEP
        }
    };

    gload(0);
    lstore(0, 0);
    __syncthreads();
    int buf = 0;
    for (int kt = 0; kt + 1 < nk; ++kt) {
        gload(kt + 1);
        __builtin_amdgcn_sched_barrier(0);         // the fetch goes first: it has the whole step to arrive
        compute(buf, [&]() {
            // staging between the two halves of the MFMAs costs less of them than staging behind the
            // last one (measured: 0.7 %); the fetch has had half a step (64 MFMAs) to arrive
            __builtin_amdgcn_sched_barrier(0);
            lstore(buf ^ 1, kt + 1);
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
        buf ^= 1;
    }
    compute(buf, []() {});

    // ---- epilogue: register r of a 32x32 block is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32.
    // Buffer stores: the row of a register is a wave-uniform offset from the tile's first row, the lane's
    // own offset (its column, its half of the rows) never changes -- no per-store address arithmetic on the
    // vector ALU, which would take issue slots from the MFMAs of the co-resident workgroups.  Rows past
    // the end of C fall outside the window and are dropped by the hardware; a lane whose column does not
    // exist is sent outside the window.
    // The window is the tile's own rows (less than 2 GB: the entry point checks), so the offset that sends a
    // lane outside it cannot wrap around 32 bits when the row offset is added.
    // C_l = centre - radius, C_u = centre + radius
#pragma unroll
    for (int a = 0; a < MBM; ++a)
#pragma unroll
        for (int b = 0; b < MBN; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float c = cl[a][b][r], rd = cu[a][b][r];      // 2 M and 2 R
                cl[a][b][r] = 0.5f * (c - rd);
                cu[a][b][r] = 0.5f * (c + rd);
            }
    const size_t c_bytes = (size_t)min(M - m0, BM) * g.N * 4;
    if constexpr (EPI == EPI_RELU) {
#pragma clang fp contract(off)          // the lines are formed with the reference's separate roundings
        static_assert(NQ >= 0, "the dual norm of the perturbation");
        const ReluArgs *ra = &epi;
        float nl[MBN], nu[MBN];
#pragma unroll
        for (int b = 0; b < MBN; ++b) {
            nl[b] = nu[b] = 0.f;
#pragma unroll
            for (int a = 0; a < MBM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    nl[b] = nacc<NQ>(nl[b], cl[a][b][r], qv);
                    nu[b] = nacc<NQ>(nu[b], cu[a][b][r], qv);
                }
            nl[b] = ncomb<NQ>(nl[b], __shfl_xor(nl[b], 32, 64));
            nu[b] = ncomb<NQ>(nu[b], __shfl_xor(nu[b], 32, 64));
        }
        // the constant terms are read before the barrier and written behind it: out_lb may be g.Dl
        float lb0[MBN], ub0[MBN];
#pragma unroll
        for (int b = 0; b < MBN; ++b) {
            const int col = n0 + (wn * MBN + b) * 32 + fi;
            const size_t o = (size_t)m_blk * g.N + min(col, g.N - 1);
            lb0[b] = g.Dl[o];
            ub0[b] = g.Du[o];
        }
        __syncthreads();                               // every wavefront has read its last fragments: LDS is free
        float *red = smem;                             // [wm][l, u][BN columns]
        if (fh == 0) {
#pragma unroll
            for (int b = 0; b < MBN; ++b) {
                red[(wm * 2 + 0) * BN + (wn * MBN + b) * 32 + fi] = nl[b];
                red[(wm * 2 + 1) * BN + (wn * MBN + b) * 32 + fi] = nu[b];
            }
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < MBN; ++b) {
            const int cb = (wn * MBN + b) * 32 + fi, col = n0 + cb;
            const float tl = ncomb<NQ>(red[(0 * 2 + 0) * BN + cb], red[(1 * 2 + 0) * BN + cb]);
            const float tu = ncomb<NQ>(red[(0 * 2 + 1) * BN + cb], red[(1 * 2 + 1) * BN + cb]);
            // l = lb + (-eps * norm), two roundings as Bounds.concretize has them (Bounds.py:313, 324)
            const float l = __fadd_rn(lb0[b], __fmul_rn(-ra->eps, nfin<NQ>(tl, qv)));
            const float u = __fadd_rn(ub0[b], __fmul_rn(ra->eps, nfin<NQ>(tu, qv)));
            // the two lines of Bounds.relu (Bounds.py:921-963) and their constant terms as Bounds.add_linear forms
            // them (Bounds.py:378, :381: (b - x0) * k + y0, b the same-side constant for a positive slope) --
            // relax_point<RELU> of the relaxation kernels written out on scalars, so that nothing goes through memory
            float klo, kup, x0up = 0.f;
            if (u < 0.f) {
                klo = kup = 0.f;
            } else if (l > 0.f) {
                klo = kup = 1.f;
            } else {
                kup = u / ((u - l) + TINY);
                x0up = l;
                klo = fabsf(u) > fabsf(l) ? 1.f : 0.f;
            }
            const float olb = ((klo > 0.f ? lb0[b] : ub0[b]) - 0.f) * klo + 0.f;
            const float oub = ((kup > 0.f ? ub0[b] : lb0[b]) - x0up) * kup + 0.f;
            if (wm == 0 && fh == 0 && col < g.N) {
                const size_t o = (size_t)m_blk * g.N + col;
                ra->out_lb[o] = olb;
                ra->out_ub[o] = oub;
            }
#pragma unroll
            for (int a = 0; a < MBM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    cl[a][b][r] *= klo;                 // both slopes are >= 0: each side keeps its own coefficients
                    cu[a][b][r] *= kup;
                }
        }
    }
    if constexpr (EPI == EPI_ROWNORM) {
        const RowNormArgs *rn = &epi;
        static_assert(MBM == 1, "whole rows: one 32-row block per wavefront");
        const unsigned row_b = (unsigned)g.N * 4u;
        unsigned vo[MBN];
#pragma unroll
        for (int b = 0; b < MBN; ++b) vo[b] = (unsigned)(4 * fh) * row_b + (unsigned)((wn * MBN + b) * 32 + fi) * 4u;
        auto row_off = [&](int r) { return (unsigned)(wm * 32 + 8 * (r / 4) + (r % 4)) * row_b; };
        // ---- the added object: its rows for this tile (a tile lies inside one position: dim_in % 64 == 0)
        if (rn->res_l) {
            long long first = m0;
            bool there = true;
            if (rn->positions) {
                const int q = m0 / rn->dim_in, bb = q / rn->length, pos = q % rn->length;
                int slot = -1;
                for (int i = 0; i < rn->words; ++i)
                    if (rn->positions[bb * rn->words + i] == pos) slot = i;
                slot = __builtin_amdgcn_readfirstlane(slot);     // the same in every lane: keeps the descriptors in scalar registers
                there = slot >= 0;
                first = ((long long)bb * rn->words + slot) * rn->dim_in + m0 % rn->dim_in;
            }
            if (there) {
                const __amdgpu_buffer_rsrc_t wrl = window(rn->res_l + (size_t)first * g.N, c_bytes);
                const __amdgpu_buffer_rsrc_t wru = window(rn->res_u + (size_t)first * g.N, c_bytes);
#pragma unroll
                for (int b = 0; b < MBN; ++b) {
                    float tl[16], tu[16];
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        tl[r] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wrl, vo[b], row_off(r), 0));
                        tu[r] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wru, vo[b], row_off(r), 0));
                    }
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        cl[0][b][r] += tl[r];          // one fp32 add, as Bounds.add rounds it
                        cu[0][b][r] += tu[r];
                    }
                }
            }
        }
        // ---- row sums: the lane's MBN columns, the 32 lanes of its half, the two wavefronts that share the rows
        float sl[16], su[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sl[r] = cl[0][0][r];
            su[r] = cu[0][0][r];
#pragma unroll
            for (int b = 1; b < MBN; ++b) {
                sl[r] += cl[0][b][r];
                su[r] += cu[0][b][r];
            }
        }
#define FAITH_STEP(MSK)                                  \
    _Pragma("unroll") for (int r = 0; r < 16; ++r) {    \
        sl[r] += lane_xor<MSK>(sl[r]);                  \
        su[r] += lane_xor<MSK>(su[r]);                  \
    }
        FAITH_STEP(1) FAITH_STEP(2) FAITH_STEP(4) FAITH_STEP(8) FAITH_STEP(16)
#undef FAITH_STEP
        __syncthreads();                               // every wavefront has read its last fragments: LDS is free
        float *red = smem;                             // [wn][l, u][64 rows of the tile]
        if (fi == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = wm * 32 + 8 * (r / 4) + 4 * fh + (r % 4);
                red[(wn * 2 + 0) * 64 + row] = sl[r];
                red[(wn * 2 + 1) * 64 + row] = su[r];
            }
        }
        __syncthreads();
        const float inv = 1.f / (float)g.N;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = wm * 32 + 8 * (r / 4) + 4 * fh + (r % 4);
            sl[r] = (red[(0 * 2 + 0) * 64 + row] + red[(1 * 2 + 0) * 64 + row]) * inv;     // mean of the lower side
            su[r] = (red[(0 * 2 + 1) * 64 + row] + red[(1 * 2 + 1) * 64 + row]) * inv;
        }
        // ---- centre on the other side's mean, scale by the weight split by sign, store
        const __amdgpu_buffer_rsrc_t wol = window(rn->out_l + (size_t)m0 * g.N, c_bytes);
        const __amdgpu_buffer_rsrc_t wou = window(rn->out_u + (size_t)m0 * g.N, c_bytes);
#pragma unroll
        for (int b = 0; b < MBN; ++b) {
            float sp = 1.f, sn = 0.f;
            if (rn->weight) {
                const float wgt = rn->weight[(wn * MBN + b) * 32 + fi];
                sp = wgt > 0.f ? wgt : 0.f * wgt;
                sn = wgt - sp;
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float c_lo = cl[0][b][r] - su[r], c_up = cu[0][b][r] - sl[r];
                const float ol = rn->weight ? c_lo * sp + c_up * sn : c_lo;
                const float ou = rn->weight ? c_lo * sn + c_up * sp : c_up;
                const unsigned so = __builtin_amdgcn_readfirstlane(row_off(r));      // a scalar operand, stated as one
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(ol), wol, vo[b], so, 2);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(ou), wou, vo[b], so, 2);
            }
        }
        return;
    }
    const __amdgpu_buffer_rsrc_t wcl = window(g.Cl + (size_t)m0 * g.N, c_bytes);
    const __amdgpu_buffer_rsrc_t wcu = window(g.Cu + (size_t)m0 * g.N, c_bytes);
    const unsigned row_b = (unsigned)g.N * 4u;
#pragma unroll
    for (int b = 0; b < MBN; ++b) {
        const int col = n0 + (wn * MBN + b) * 32 + fi;
        const unsigned vo = col < g.N ? (unsigned)(4 * fh) * row_b + (unsigned)col * 4u : 0x80000000u;
#pragma unroll
        for (int a = 0; a < MBM; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned so = (unsigned)((wm * MBM + a) * 32 + 8 * (r / 4) + (r % 4)) * row_b;
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(cl[a][b][r]), wcl, vo, so, 2 /* non-temporal */);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(cu[a][b][r]), wcu, vo, so, 2);
            }
        }
    }
    if constexpr (NQ >= 0 && EPI == EPI_PLAIN) {
        // the lane's 16 MBM rows of each of its columns, in register order (a fixed order: the result does not
        // depend on scheduling)
#pragma unroll
        for (int b = 0; b < MBN; ++b)
#pragma unroll
            for (int a = 0; a < MBM; ++a)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    pl[b] = nacc<NQ>(pl[b], cl[a][b][r], qv);
                    pu[b] = nacc<NQ>(pu[b], cu[a][b][r], qv);
                }
    }
}

// One tile per workgroup: workgroups are dealt round-robin to the XCDs, so the N-tiles that share an M-block
// get ids 8 apart and meet in one L2.
template <bool EXACT, int MBM, int MBN>
__device__ __forceinline__ void signsplit_gemm_body(const GemmArgs &g, float *smem, const int pid) {
    constexpr int BM = 64 * MBM, BN = 64 * MBN;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int mblks = (g.Mw + BM - 1) / BM;
    const int xcd = pid % XCDS, local = pid / XCDS;
    const int m_blk = (local / tiles_n) * XCDS + xcd;
    const int n_blk = local % tiles_n;
    if (m_blk >= mblks) return;
    signsplit_gemm_tile<EXACT, MBM, MBN>(g, smem, m_blk, n_blk);
}

}  // namespace

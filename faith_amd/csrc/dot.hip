// McCormick bounds of the attention scores  z[i, j] = sum_k x[i, k] * y[j, k]  on fp32 MFMA.
//
// Arithmetic of the reference's Bounds.ori_dot_product with get_bounds_xy
// (Transformer_Verification_Code/Verifiers/Bounds.py:666-688, :710-823).  With the concrete
// intervals [l_x, u_x] of x and [l_y, u_y] of y, the planes are
//     x*y >= a_l x + b y - a_l b,   x*y <= a_u x + b y - a_u b,   a_l = l_y, a_u = u_y, b = l_x
// (b = l_x on both sides, as the reference has it), and each plane is pushed through the linear
// bounds of x and y by the sign of its coefficient.  For a fixed perturbation coordinate m this
// is one [Lx x Ly] tile with a reduction over d:
//   z_lw[i,m,j] = sum_k  xlw[i,m,k] a_l+[j,k] + xuw[i,m,k] a_l-[j,k] + b+[i,k] ylw[j,m,k] + b-[i,k] yuw[j,m,k]
//   z_uw[i,m,j] = sum_k  xuw[i,m,k] a_u+[j,k] + xlw[i,m,k] a_u-[j,k] + b+[i,k] yuw[j,m,k] + b-[i,k] ylw[j,m,k]
// i.e. eight MFMA products per K-pair into two accumulators.  Rows (i) come from x and b, columns
// (j) from a and y, so the accumulator tile is already laid out as z[i, m, j..]: lanes run along j
// and every store is a 128-byte run.  Neither the [Lx, D, d, Ly] broadcast the PyTorch code
// materialises nor the transposed add of its y-terms exists here.
//
// Tiling: workgroup = 4 wavefronts on a 128 x 128 (i x j) tile of one (head, m); wavefront tile
// 64 x 64 (2 x 2 blocks of v_mfma_f32_32x32x2_f32, for each of z_lw and z_uw).  K-step 8:
// seven operand tiles [128 x 8] per step (xlw, xuw, b | a_l, a_u, ylw, yuw) = 28 KB, double
// buffered = 56 KB, so two workgroups share a CU.  Rows are 8 floats with the two 16-byte halves
// swapped on every other group of four rows, which makes both the 16-byte stores and the 16-byte
// fragment reads bank-conflict free without padding.  a / b are split by sign after the LDS
// read (v_max / v_min); they are staged from the concretization results, unsplit.
//
// The constant terms z_lb / z_ub ([Lx, Ly] per head, 1/D_in of the work, O(1) cancelling terms)
// are summed in double by a small kernel.
#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TI = 128, TJ = 128, BK = 8;
constexpr int NTHREADS = 256;
constexpr int TILE = 128 * BK;            // floats per operand tile

struct DotArgs {
    const float *xlw, *xuw, *ylw, *yuw;   // [B, Lx, D, d], [B, Ly, D, d]
    const float *xlb, *xub, *ylb, *yub;   // [B, Lx, d], [B, Ly, d]
    const float *x_l, *y_l, *y_u;         // concrete intervals: b = x_l, a_l = y_l, a_u = y_u
    float *zlw, *zuw;                     // [B, Lx, D, Ly]
    float *zlb, *zub;                     // [B, Lx, Ly]
    int B, Lx, Ly, D, d;
};

__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 pos4(float4 v) {
    return make_float4(fmaxf(v.x, 0.f), fmaxf(v.y, 0.f), fmaxf(v.z, 0.f), fmaxf(v.w, 0.f));
}
__device__ __forceinline__ float4 neg4(float4 v) {
    return make_float4(fminf(v.x, 0.f), fminf(v.y, 0.f), fminf(v.z, 0.f), fminf(v.w, 0.f));
}

// position of 16-byte half `c` (0 / 1) of row `row` inside an [128 x 8] tile
__device__ __forceinline__ int swz(int row, int c) { return row * BK + 4 * (c ^ ((row >> 2) & 1)); }

enum { XL = 0, XU, BT, AL, AU, YL, YU, NOPS };

// Persistent: the grid is sized to the machine (two workgroups per CU) and every workgroup walks
// tiles pid, pid + grid, ...  The walk is ONE software pipeline over (tile, K-step): the global
// loads of the next step -- the first K-step of the next tile included -- are issued before the
// MFMAs of the current step, and the accumulator stores of a finished tile are issued while
// those loads are in flight, so neither the head nor the tail of a tile leaves the MFMA pipe idle.
//
// VP = false: scores path, y is [B, Ly, D, d] (reduction axis contiguous, like x).
// VP = true : context path (probs . value): y is the value bound object in its own natural layout
//   [B, d, D, Ly] -- the reduction axis (key position) is the slow one and j is contiguous --
//   and so are its concrete bounds [B, d, Ly].  The y-side tiles are then staged as [k][j]
//   (16-byte loads along j, conflict-free) and their fragments read with four 4-byte LDS reads.
template <bool VP>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
dot_w(const DotArgs g, const int total_tiles) {
    __shared__ float sm[2][NOPS][TILE];

    const int ti = (g.Lx + TI - 1) / TI, tj = (g.Ly + TJ - 1) / TJ;
    const int d = g.d;
    const int nk = (d + BK - 1) / BK;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int wi = wv / 2, wj = wv % 2;
    const int fi = lane % 32, fh = lane / 32;

    // ---- staging: one float4 per operand per thread per K-step
    const int srow = tid / 2, sc = tid % 2;
    const int sdst = swz(srow, sc);
    const int vk = tid / 32, vj = (tid % 32) * 4;          // VP: this thread's (k, j..j+3) of a y-side tile
    const int ydst = VP ? vk * TJ + vj : sdst;
    // element offsets of this thread's source rows (32-bit: the entry point checks the sizes);
    // xlw / xuw share one, ylw / yuw share one, a_l / a_u share one
    unsigned ox, oy, obt, oa;
    bool y_in = true;                                      // VP: columns past Ly are staged as zeros
    float4 pre[NOPS];
    auto point_at = [&](int tile) {
        int q = tile;
        const int j0 = (q % tj) * TJ;  q /= tj;
        const int i0 = (q % ti) * TI;  q /= ti;
        const int m = q % g.D, t = q / g.D;
        const int irow = min(i0 + srow, g.Lx - 1);         // clamped rows are never stored
        ox = ((unsigned)(t * g.Lx + irow) * g.D + m) * d + sc * 4;
        obt = (unsigned)(t * g.Lx + irow) * d + sc * 4;
        if (VP) {
            y_in = j0 + vj < g.Ly;                         // Ly % 4 == 0
            oy = ((unsigned)(t * d + vk) * g.D + m) * g.Ly + j0 + vj;
            oa = (unsigned)(t * d + vk) * g.Ly + j0 + vj;
        } else {
            const int jrow = min(j0 + srow, g.Ly - 1);
            oy = ((unsigned)(t * g.Ly + jrow) * g.D + m) * d + sc * 4;
            oa = (unsigned)(t * g.Ly + jrow) * d + sc * 4;
        }
    };
    auto gload = [&](int kt) {
        const int k = kt * BK;
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
        const bool x_ok = k + sc * 4 < d;                  // d % 4 == 0: a float4 is all in or all out
        pre[XL] = x_ok ? ld4(g.xlw + ox + k) : zero;
        pre[XU] = x_ok ? ld4(g.xuw + ox + k) : zero;
        pre[BT] = x_ok ? ld4(g.x_l + obt + k) : zero;
        if (VP) {
            const bool y_ok = y_in && k + vk < d;
            const unsigned ky = (unsigned)k * g.D * g.Ly, ka = (unsigned)k * g.Ly;
            pre[AL] = y_ok ? ld4(g.y_l + oa + ka) : zero;
            pre[AU] = y_ok ? ld4(g.y_u + oa + ka) : zero;
            pre[YL] = y_ok ? ld4(g.ylw + oy + ky) : zero;
            pre[YU] = y_ok ? ld4(g.yuw + oy + ky) : zero;
        } else {
            pre[AL] = x_ok ? ld4(g.y_l + oa + k) : zero;
            pre[AU] = x_ok ? ld4(g.y_u + oa + k) : zero;
            pre[YL] = x_ok ? ld4(g.ylw + oy + k) : zero;
            pre[YU] = x_ok ? ld4(g.yuw + oy + k) : zero;
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int o = 0; o < NOPS; ++o)
            *reinterpret_cast<float4 *>(&sm[buf][o][(o == XL || o == XU || o == BT) ? sdst : ydst]) = pre[o];
    };
    // y-side fragment of block b: four K values of column j; [j][k] tile -> one 16-byte read,
    // [k][j] tile (VP) -> four 4-byte reads, lanes along j
    auto yfrag = [&](int buf, int o, int b) -> float4 {
        if (VP) {
            const float *p = &sm[buf][o][(4 * fh) * TJ + wj * 64 + b * 32 + fi];
            return make_float4(p[0], p[TJ], p[2 * TJ], p[3 * TJ]);
        }
        return *reinterpret_cast<const float4 *>(&sm[buf][o][swz(wj * 64 + b * 32 + fi, fh)]);
    };

    int fa[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) fa[s] = swz(wi * 64 + s * 32 + fi, fh);

    floatx16 cl[2][2], cu[2][2];
    int tile = blockIdx.x;
    if (tile >= total_tiles) return;
    point_at(tile);
    gload(0);
    lstore(0);
    __syncthreads();
    int buf = 0;
    for (; tile < total_tiles; tile += gridDim.x) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;
        const int next_tile = tile + gridDim.x;
        const bool has_next = next_tile < total_tiles;
        for (int kt = 0; kt < nk; ++kt) {
            const bool last = kt + 1 == nk;
            if (!last) {
                gload(kt + 1);
            } else if (has_next) {
                point_at(next_tile);
                gload(0);
            }
            float4 xl[2], xu[2], bp[2], bn[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                xl[s] = *reinterpret_cast<const float4 *>(&sm[buf][XL][fa[s]]);
                xu[s] = *reinterpret_cast<const float4 *>(&sm[buf][XU][fa[s]]);
                const float4 bt = *reinterpret_cast<const float4 *>(&sm[buf][BT][fa[s]]);
                bp[s] = pos4(bt);
                bn[s] = neg4(bt);
            }
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const float4 al = yfrag(buf, AL, b), au = yfrag(buf, AU, b);
                const float4 yl = yfrag(buf, YL, b), yu = yfrag(buf, YU, b);
                const float4 alp = pos4(al), aln = neg4(al), aup = pos4(au), aun = neg4(au);
#define FAITH_DOT_STEP(c)                                   \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cl[a][b] = mfma(xl[a].c, alp.c, cl[a][b]);          \
        cu[a][b] = mfma(xu[a].c, aup.c, cu[a][b]);          \
    }                                                       \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cl[a][b] = mfma(xu[a].c, aln.c, cl[a][b]);          \
        cu[a][b] = mfma(xl[a].c, aun.c, cu[a][b]);          \
    }                                                       \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cl[a][b] = mfma(bp[a].c, yl.c, cl[a][b]);           \
        cu[a][b] = mfma(bp[a].c, yu.c, cu[a][b]);           \
    }                                                       \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cl[a][b] = mfma(bn[a].c, yu.c, cl[a][b]);           \
        cu[a][b] = mfma(bn[a].c, yl.c, cu[a][b]);           \
    }
                FAITH_DOT_STEP(x)
                FAITH_DOT_STEP(y)
                FAITH_DOT_STEP(z)
                FAITH_DOT_STEP(w)
#undef FAITH_DOT_STEP
            }
            if (!last) {
                lstore(buf ^ 1);
                __syncthreads();
                buf ^= 1;
            }
        }
        {
            // ---- z[t, i, m, j]; register r of a block is row 8*(r/4) + 4*(lane/32) + r%4.
            // Issued while the first K-step of the next tile is on its way.
            int q = tile;
            const int j0 = (q % tj) * TJ;  q /= tj;
            const int i0 = (q % ti) * TI;  q /= ti;
            const int m = q % g.D, t = q / g.D;
            const unsigned rs = (unsigned)g.D * g.Ly;                     // one step in i
            const int ib = i0 + wi * 64 + 4 * fh;
            const unsigned ob = ((unsigned)(t * g.Lx + ib) * g.D + m) * g.Ly + j0 + wj * 64 + fi;
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                if (j0 + wj * 64 + b * 32 + fi >= g.Ly) continue;
#pragma unroll
                for (int a = 0; a < 2; ++a) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int di = a * 32 + 8 * (r / 4) + (r % 4);
                        if (ib + di < g.Lx) {
                            const unsigned o = ob + di * rs + b * 32;
                            __builtin_nontemporal_store(cl[a][b][r], &g.zlw[o]);
                            __builtin_nontemporal_store(cu[a][b][r], &g.zuw[o]);
                        }
                    }
                }
            }
        }
        if (has_next) lstore(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
}

// Any-shape coefficient kernel (d not a multiple of 4, unaligned pointers): one thread per
// (i, m, j), products and sums in double.
template <bool VP>
__global__ void __launch_bounds__(256) dot_w_simple(const DotArgs g) {
    const size_t total = (size_t)g.B * g.Lx * g.D * g.Ly;
    for (size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (size_t)gridDim.x * 256) {
        const int j = idx % g.Ly;
        const int m = (idx / g.Ly) % g.D;
        const int i = (idx / ((size_t)g.Ly * g.D)) % g.Lx;
        const int t = idx / ((size_t)g.Ly * g.D * g.Lx);
        const float *xl = g.xlw + ((size_t)(t * g.Lx + i) * g.D + m) * g.d;
        const float *xu = g.xuw + ((size_t)(t * g.Lx + i) * g.D + m) * g.d;
        // y element (j, m, k): scores path [t, j, m, k]; context path [t, k, m, j]
        const size_t ybase = VP ? ((size_t)t * g.d * g.D + m) * g.Ly + j : ((size_t)(t * g.Ly + j) * g.D + m) * g.d;
        const size_t ystep = VP ? (size_t)g.D * g.Ly : 1;
        const size_t abase = VP ? (size_t)t * g.d * g.Ly + j : (size_t)(t * g.Ly + j) * g.d;
        const size_t astep = VP ? g.Ly : 1;
        const float *bt = g.x_l + (size_t)(t * g.Lx + i) * g.d;
        double sl = 0.0, su = 0.0;
        for (int k = 0; k < g.d; ++k) {
            const float yl = g.ylw[ybase + k * ystep], yu = g.yuw[ybase + k * ystep];
            const float al = g.y_l[abase + k * astep], au = g.y_u[abase + k * astep];
            const double bp = fmaxf(bt[k], 0.f), bn = fminf(bt[k], 0.f);
            const double alp = fmaxf(al, 0.f), aln = fminf(al, 0.f);
            const double aup = fmaxf(au, 0.f), aun = fminf(au, 0.f);
            sl += xl[k] * alp + xu[k] * aln + bp * yl + bn * yu;
            su += xu[k] * aup + xl[k] * aun + bp * yu + bn * yl;
        }
        g.zlw[idx] = (float)sl;
        g.zuw[idx] = (float)su;
    }
}

// Constant terms (Bounds.py:761-762 gamma, :804-807, :815-818): a workgroup owns a 16 x 16 tile of
// (i, j) of one head, stages the seven [16 x d-chunk] operand rows in LDS and sums in double.
constexpr int BT_T = 16, BT_K = 64;
template <bool VP>
__global__ void __launch_bounds__(256) dot_b(const DotArgs g) {
    __shared__ float sx[3][BT_T][BT_K + 1];     // b (= l_x), xlb, xub
    __shared__ float sy[4][BT_T][BT_K + 1];     // a_l, a_u, ylb, yub
    const int ti = (g.Lx + BT_T - 1) / BT_T, tj = (g.Ly + BT_T - 1) / BT_T;
    int pid = blockIdx.x;
    const int j0 = (pid % tj) * BT_T;  pid /= tj;
    const int i0 = (pid % ti) * BT_T;  pid /= ti;
    const int t = pid;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;     // output (i0 + ty, j0 + tx)
    double sl = 0.0, su = 0.0;
    for (int k0 = 0; k0 < g.d; k0 += BT_K) {
        for (int e = threadIdx.x; e < BT_T * BT_K; e += 256) {
            const int r = e / BT_K, k = e % BT_K;
            const bool kin = k0 + k < g.d;
            const bool xin = kin && i0 + r < g.Lx, yin = kin && j0 + r < g.Ly;
            const size_t xo = (size_t)(t * g.Lx + i0 + r) * g.d + k0 + k;
            const size_t yo = VP ? (size_t)(t * g.d + k0 + k) * g.Ly + j0 + r : (size_t)(t * g.Ly + j0 + r) * g.d + k0 + k;
            sx[0][r][k] = xin ? g.x_l[xo] : 0.f;
            sx[1][r][k] = xin ? g.xlb[xo] : 0.f;
            sx[2][r][k] = xin ? g.xub[xo] : 0.f;
            sy[0][r][k] = yin ? g.y_l[yo] : 0.f;
            sy[1][r][k] = yin ? g.y_u[yo] : 0.f;
            sy[2][r][k] = yin ? g.ylb[yo] : 0.f;
            sy[3][r][k] = yin ? g.yub[yo] : 0.f;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < BT_K; ++k) {
            const double bt = sx[0][ty][k], xlb = sx[1][ty][k], xub = sx[2][ty][k];
            const double al = sy[0][tx][k], au = sy[1][tx][k], ylb = sy[2][tx][k], yub = sy[3][tx][k];
            const double bp = bt > 0 ? bt : 0, bn = bt < 0 ? bt : 0;
            sl += -al * bt + (al > 0 ? al * xlb : al * xub) + bp * ylb + bn * yub;
            su += -au * bt + (au > 0 ? au * xub : au * xlb) + bp * yub + bn * ylb;
        }
        __syncthreads();
    }
    const int i = i0 + ty, j = j0 + tx;
    if (i < g.Lx && j < g.Ly) {
        const size_t o = ((size_t)t * g.Lx + i) * g.Ly + j;
        g.zlb[o] = (float)sl;
        g.zub[o] = (float)su;
    }
}

// dim_in == 1: the reference switches to plain interval arithmetic on the constant terms and
// returns zero coefficients (Bounds.py:711-721).
template <bool VP>
__global__ void __launch_bounds__(256) dot_interval(const DotArgs g) {
    const size_t total = (size_t)g.B * g.Lx * g.Ly;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int j = idx % g.Ly;
    const int i = (idx / g.Ly) % g.Lx;
    const int t = idx / ((size_t)g.Ly * g.Lx);
    const size_t xo = (size_t)(t * g.Lx + i) * g.d;
    const size_t yo = VP ? (size_t)t * g.d * g.Ly + j : (size_t)(t * g.Ly + j) * g.d, ys = VP ? g.Ly : 1;
    float lo = 0.f, hi = 0.f;
    for (int k = 0; k < g.d; ++k) {
        const float l1 = g.xlb[xo + k], u1 = g.xub[xo + k], l2 = g.ylb[yo + k * ys], u2 = g.yub[yo + k * ys];
        const float c1 = l1 * l2, c2 = l1 * u2, c3 = u1 * l2, c4 = u1 * u2;
        lo += fminf(fminf(c1, c2), fminf(c3, c4));
        hi += fmaxf(fmaxf(c1, c2), fmaxf(c3, c4));
    }
    g.zlb[idx] = lo;
    g.zub[idx] = hi;
    g.zlw[idx] = 0.f;      // [B, Lx, 1, Ly] has the same linear index
    g.zuw[idx] = 0.f;
}

// Shared body of the two entry points.  For the context path (VP) `d` is the number of key positions
// (the reduction length) and `Ly` the width of the value vectors; y_* are the value bounds in their
// natural layout [B, d, D, Ly] / [B, d, Ly].
template <bool VP>
int dot_entry(const char *who, float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb, const float *x_ub,
              const float *y_lb, const float *y_ub, const float *x_lw, const float *x_uw, const float *y_lw,
              const float *y_uw, float *z_lb, float *z_ub, float *z_lw, float *z_uw, int B, int Lx, int Ly, int d, int D,
              float epsilon, int q, int words, void *stream) {
    FAITH_NOT_NULL(x_l); FAITH_NOT_NULL(y_l); FAITH_NOT_NULL(x_u); FAITH_NOT_NULL(y_u);
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub);
    FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_NOT_NULL(z_lb); FAITH_NOT_NULL(z_ub); FAITH_NOT_NULL(z_lw); FAITH_NOT_NULL(z_uw);
    FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_ALIGNED4(z_lw); FAITH_ALIGNED4(z_uw); FAITH_ALIGNED4(z_lb); FAITH_ALIGNED4(z_ub);
    FAITH_REQUIRE(B > 0 && Lx > 0 && Ly > 0 && d > 0 && D > 0, FAITH_ERR_SHAPE,
                  "%s: batch=%d rows of x=%d columns of z=%d reduction length=%d dim_in=%d must be positive", who, B,
                  Lx, Ly, d, D);
    const long long nw = (long long)B * Lx * D * Ly;
    const long long nx = (long long)B * Lx * D * d, ny = (long long)B * Ly * D * d;
    FAITH_REQUIRE((long long)B * (Lx > Ly ? Lx : Ly) * D <= 0x7fffffffLL && (long long)B * d * D <= 0x7fffffffLL,
                  FAITH_ERR_SHAPE, "%s: batch*length*dim_in exceeds 2^31", who);

    hipStream_t st = static_cast<hipStream_t>(stream);
    DotArgs g{x_lw, x_uw, y_lw, y_uw, x_lb, x_ub, y_lb, y_ub, x_l, y_l, y_u, z_lw, z_uw, z_lb, z_ub, B, Lx, Ly, D, d};
    if (D == 1) {
        const long long n = (long long)B * Lx * Ly;
        hipLaunchKernelGGL(dot_interval<VP>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, g);
        return faith::check_launch(who);
    }

    // concrete intervals of both operands (Bounds.py:725-726); x_u is produced because the reference
    // interface exposes it, the planes do not use it.  One launch when both objects have the same
    // [D, H] shape (always on the scores path).
    const int y_rows = VP ? B * d : B * Ly, y_h = VP ? Ly : d;
    int rc;
    if (y_h == d) {
        rc = faith::concretize_pair(x_lb, x_ub, x_lw, x_uw, x_l, x_u, B * Lx, y_lb, y_ub, y_lw, y_uw, y_l, y_u, y_rows,
                                    D, d, epsilon, q, words, stream);
    } else {
        rc = faith_concretize(x_lb, x_ub, x_lw, x_uw, x_l, x_u, B * Lx, D, d, epsilon, q, words,
                              FAITH_LAYOUT_NATURAL, stream);
        if (rc == FAITH_OK)
            rc = faith_concretize(y_lb, y_ub, y_lw, y_uw, y_l, y_u, y_rows, D, y_h, epsilon, q, words,
                                  FAITH_LAYOUT_NATURAL, stream);
    }
    if (rc != FAITH_OK) return rc;

    hipLaunchKernelGGL(dot_b<VP>, dim3((unsigned)((long long)B * ((Lx + BT_T - 1) / BT_T) * ((Ly + BT_T - 1) / BT_T))),
                       dim3(256), 0, st, g);

    const bool fast = (d % 4 == 0) && (!VP || Ly % 4 == 0) && faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) &&
                      faith::aligned(y_lw, 16) && faith::aligned(y_uw, 16) && faith::aligned(x_l, 16) &&
                      faith::aligned(y_l, 16) && faith::aligned(y_u, 16) && nw < 0xffffffffLL && nx < 0xffffffffLL &&
                      ny < 0xffffffffLL;
    if (fast) {
        const long long tiles = (long long)B * D * ((Lx + TI - 1) / TI) * ((Ly + TJ - 1) / TJ);
        FAITH_REQUIRE(tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: too many tiles", who);
        const long long resident = 2LL * faith::compute_units();      // 56 KB of LDS each: two per CU
        hipLaunchKernelGGL(dot_w<VP>, dim3((unsigned)(tiles < resident ? tiles : resident)), dim3(NTHREADS), 0, st, g,
                           (int)tiles);
    } else {
        const long long blocks = (nw + 255) / 256;
        hipLaunchKernelGGL(dot_w_simple<VP>, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, st, g);
    }
    return faith::check_launch(who);
}

}  // namespace

extern "C" int faith_dot_product_verification_QK(float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                                                 const float *x_ub, const float *y_lb, const float *y_ub,
                                                 const float *x_lw, const float *x_uw, const float *y_lw,
                                                 const float *y_uw, float *z_lb, float *z_ub, float *z_lw,
                                                 float *z_uw, int batch_size, int length_x, int length_y,
                                                 int dim_out, int dim_in, float epsilon, int q, int words,
                                                 void *stream) {
    return dot_entry<false>("faith_dot_product_verification_QK", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw,
                            y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size, length_x, length_y, dim_out, dim_in, epsilon,
                            q, words, stream);
}

extern "C" int faith_dot_product_verification_V(float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                                                const float *x_ub, const float *y_lb, const float *y_ub,
                                                const float *x_lw, const float *x_uw, const float *y_lw,
                                                const float *y_uw, float *z_lb, float *z_ub, float *z_lw,
                                                float *z_uw, int batch_size, int length_x, int length_k, int dim_out,
                                                int dim_in, float epsilon, int q, int words, void *stream) {
    return dot_entry<true>("faith_dot_product_verification_V", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw,
                           y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size, length_x, dim_out, length_k, dim_in, epsilon,
                           q, words, stream);
}

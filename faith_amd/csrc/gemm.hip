// Sign-split affine bound propagation  y = x @ W^T (+ bias)  on fp32 MFMA.
//
// Arithmetic of the reference's Bounds.ori_matmul + add
// (Transformer_Verification_Code/Verifiers/Bounds.py:397-413, :383-395):
//     C_l = A_l @ W+ + A_u @ W-        C_u = A_u @ W+ + A_l @ W-
// with W+ = max(W, 0), W- = min(W, 0) (value-identical to W*(W>0), W - W+).
// A_l, A_u are the bound rows ([rows*D_in, H] for lw/uw, [rows, H] for lb/ub, both K-contiguous),
// W is [N, H] as nn.Linear stores it, so both operands stream along K.
//
// Computed in centre / radius form: W+ + W- = W and W+ - W- = |W|, so
//     C_l = M - R,   C_u = M + R,   M = ((A_l + A_u) / 2) @ W,   R = ((A_u - A_l) / 2) @ |W|
// -- TWO products per term where the formula above has four, i.e. half the MFMA time for the same
// four results.  (The kernels accumulate 2 M and 2 R from A_l + A_u and A_u - A_l and halve once per result:
// one vector instruction per staged element less, the same bits.)  The halving is exact; sum and difference
// of a coefficient pair are rounded once each, by the thread that stages them; what that adds to the rounding of the four-product form (each bound then
// carries the rounding of both operands' terms: measured 1.3 - 1.9 x its error against float64, 0.1 of
// the parity bar on the configurations) is bounded by the parity tests together with the order of summation.
//
// The reference's CUTLASS path takes the constant-term rows as trailing M-blocks of the same grid
// (tvm_kernels/cuda_kernel/mma/mma_kernel.h:251-259); here they go to the exact-accumulation
// code below instead: they are 1/D_in of the work and the only outputs whose O(1) terms cancel.
// For small problems those tiles are the leading workgroups of the MFMA launch, for large ones a
// launch of their own.
//
// Tiling (gfx950): workgroup = 4 wavefronts, macro-tile BM x BN = 128 x 128, K-step 16,
// wavefront tile 64 x 64 = 2 x 2 v_mfma_f32_32x32x2_f32 blocks for EACH of M and R
// (128 accumulator registers).  One 16-byte LDS read per operand block covers four K-pairs: 8 LDS
// reads per 32 MFMAs.
//
// On this part every vector-ALU instruction a wavefront issues takes its slot from the MFMA pipe,
// so the K-loop issues almost none: centres, radii and |W| are formed ONCE, by the thread that stages
// them (separate LDS tiles); global addresses are buffer addresses (a wave-uniform descriptor and
// K offset, one per-thread offset per row that never changes), and the K-step is straight-line:
// fetch of step t+1, half the MFMAs of step t, staging of step t+1, the other half, one barrier.
//
// LDS: a K-step of an operand is two [128 x 8] halves; rows are 8 floats with the two 16-byte
// pieces swapped on every other group of four rows, which makes the 16-byte stores and the
// 16-byte fragment reads bank-conflict free without padding.  4 operands (centre, radius, W, |W|) x 8 KB
// x 2 stages = 64 KB,
// two workgroups per CU.
//
// blockIdx -> tile mapping is XCD-aware: workgroups are dealt round-robin to the 8 XCDs, so
// the N-tiles that share an M-block (and with it A_l / A_u rows) are given ids 8 apart and
// meet in the same L2.
#include "gemm_tile.h"

namespace {

// ------------------------------------------------------------------ exact-accumulation kernel
// 16 x 16 outputs per workgroup, scalar loads, products and sums in double (an fp32 x fp32
// product is exact in double), one rounding at the end.  Two uses:
//  * the constant-term rows lb' / ub': 1/D_in of the work, but their terms are O(1) and cancel,
//    which is where the order of an fp32 summation shows; accumulated in double they carry no
//    summation error at all;
//  * any shape the MFMA kernel does not take (K not a multiple of 4, unaligned pointers).
// One 16 x 16 tile: M-block m_blk counts through the coefficient rows first, then the constant rows.
// smem: 3 * 16 * 17 floats.
__device__ __forceinline__ void simple_tile(const GemmArgs &g, const int m_blk, const int n_blk, float *smem) {
    float(*sl)[17] = reinterpret_cast<float(*)[17]>(smem);
    float(*su)[17] = reinterpret_cast<float(*)[17]>(smem + 16 * 17);
    float(*sw)[17] = reinterpret_cast<float(*)[17]>(smem + 2 * 16 * 17);
    const int mblk_w = (g.Mw + 15) / 16;
    const bool brows = m_blk >= mblk_w;
    const float *Al = brows ? g.Bl : g.Al, *Au = brows ? g.Bu : g.Au;
    float *Cl = brows ? g.Dl : g.Cl, *Cu = brows ? g.Du : g.Cu;
    const int M = brows ? g.Mb : g.Mw;
    const int m0 = (brows ? m_blk - mblk_w : m_blk) * 16, n0 = n_blk * 16;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    double accm = 0.0, accr = 0.0;
    for (int k0 = 0; k0 < g.K; k0 += 16) {
        const int k = k0 + tx;
        const int ra = m0 + ty, rw = n0 + ty;
        const bool ka = k < g.K;
        sl[ty][tx] = (ka && ra < M) ? Al[(size_t)ra * g.K + k] : 0.f;
        su[ty][tx] = (ka && ra < M) ? Au[(size_t)ra * g.K + k] : 0.f;
        sw[ty][tx] = (ka && rw < g.N) ? g.W[(size_t)rw * g.K + k] : 0.f;
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            // centre / radius form (see sliced_tile): two fused multiply-adds per term instead of four
            const double w = sw[tx][kk];
            const double xl = sl[ty][kk], xu = su[ty][kk];
            accm += w * (0.5 * (xl + xu));
            accr += fabs(w) * (0.5 * (xu - xl));
        }
        __syncthreads();
    }
    const int row = m0 + ty, col = n0 + tx;
    if (row < M && col < g.N) {
        // the reference adds the bias to the rounded fp32 product (Bounds.py:391-395)
        const float add = (brows && g.bias) ? g.bias[col] : 0.f;
        Cl[(size_t)row * g.N + col] = (float)(accm - accr) + add;
        Cu[(size_t)row * g.N + col] = (float)(accm + accr) + add;
    }
}

// The same arithmetic for the constant-term rows of a SMALL problem, where a 16 x 16 tile is one long
// chain of short dependent steps: an 8 x 8 tile per workgroup, the reduction in chunks of 64 with a
// quarter of each chunk per group of 64 threads (four times the workgroups, a quarter of the chain),
// the four partial sums combined in LDS.  smem: 3 * 8 * 65 floats + 2 * 4 * 64 doubles.
__device__ __forceinline__ void sliced_tile(const GemmArgs &g, const int m_blk, const int n_blk, float *smem) {
    constexpr int T = 8, KC = 64, S = 4;
    float(*sl)[KC + 1] = reinterpret_cast<float(*)[KC + 1]>(smem);
    float(*su)[KC + 1] = reinterpret_cast<float(*)[KC + 1]>(smem + T * (KC + 1));
    float(*sw)[KC + 1] = reinterpret_cast<float(*)[KC + 1]>(smem + 2 * T * (KC + 1));
    double(*red)[S][T * T] = reinterpret_cast<double(*)[S][T * T]>(smem + 3 * T * (KC + 1));        // 1560 floats in: 8-byte aligned
    const int m0 = m_blk * T, n0 = n_blk * T;
    const int ks = threadIdx.x / 64, o = threadIdx.x % 64;
    const int tx = o % T, ty = o / T;                       // output (m0 + ty, n0 + tx)
    double accm = 0.0, accr = 0.0;
    for (int k0 = 0; k0 < g.K; k0 += KC) {
        for (int e = threadIdx.x; e < T * KC; e += 256) {
            const int r = e / KC, k = e % KC;
            const bool kin = k0 + k < g.K;
            const bool ain = kin && m0 + r < g.Mb, win = kin && n0 + r < g.N;
            sl[r][k] = ain ? g.Bl[(size_t)(m0 + r) * g.K + k0 + k] : 0.f;
            su[r][k] = ain ? g.Bu[(size_t)(m0 + r) * g.K + k0 + k] : 0.f;
            sw[r][k] = win ? g.W[(size_t)(n0 + r) * g.K + k0 + k] : 0.f;
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < KC / S; ++kk) {
            const int k = ks * (KC / S) + kk;
            // xl w+ + xu w- = w m - |w| r and xu w+ + xl w- = w m + |w| r with m = (xl + xu) / 2,
            // r = (xu - xl) / 2, both exact in double: two fused multiply-adds per term instead of four
            const double w = sw[tx][k];
            const double xl = sl[ty][k], xu = su[ty][k];
            accm += w * (0.5 * (xl + xu));
            accr += fabs(w) * (0.5 * (xu - xl));
        }
        __syncthreads();
    }
    red[0][ks][o] = accm - accr;
    red[1][ks][o] = accm + accr;
    __syncthreads();
    const int row = m0 + ty, col = n0 + tx;
    if (ks == 0 && row < g.Mb && col < g.N) {
        const float add = g.bias ? g.bias[col] : 0.f;
        g.Dl[(size_t)row * g.N + col] = (float)(red[0][0][o] + red[0][1][o] + red[0][2][o] + red[0][3][o]) + add;
        g.Du[(size_t)row * g.N + col] = (float)(red[1][0][o] + red[1][1][o] + red[1][2][o] + red[1][3][o]) + add;
    }
}

// The same arithmetic for MANY constant-term rows riding in front of a small problem's MFMA tiles (the query / key /
// value layers of a batched propagation: 960 rows x 768 columns, whose 11,520 8 x 8 tiles were most of that launch):
// a 32 x 32 tile per workgroup, 2 x 2 outputs per thread, the reduction in chunks of 32 -- a sixteenth of the
// workgroups, each element of the operands staged once for 32 outputs instead of 8.  smem: 3 * 32 * 33 floats.
__device__ __forceinline__ void wide_tile(const GemmArgs &g, const int m_blk, const int n_blk, float *smem) {
    constexpr int T = 32, KC = 32;
    float(*sl)[KC + 1] = reinterpret_cast<float(*)[KC + 1]>(smem);
    float(*su)[KC + 1] = reinterpret_cast<float(*)[KC + 1]>(smem + T * (KC + 1));
    float(*sw)[KC + 1] = reinterpret_cast<float(*)[KC + 1]>(smem + 2 * T * (KC + 1));
    const int m0 = m_blk * T, n0 = n_blk * T;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;   // outputs (m0 + ty + 16 i, n0 + tx + 16 j)
    double am[2][2] = {{0.0, 0.0}, {0.0, 0.0}}, ar[2][2] = {{0.0, 0.0}, {0.0, 0.0}};
    for (int k0 = 0; k0 < g.K; k0 += KC) {
#pragma unroll
        for (int u = 0; u < T * KC / 256; ++u) {
            const int e = threadIdx.x + u * 256;
            const int r = e / KC, k = e % KC;
            const bool kin = k0 + k < g.K;
            const bool ain = kin && m0 + r < g.Mb, win = kin && n0 + r < g.N;
            sl[r][k] = ain ? g.Bl[(size_t)(m0 + r) * g.K + k0 + k] : 0.f;
            su[r][k] = ain ? g.Bu[(size_t)(m0 + r) * g.K + k0 + k] : 0.f;
            sw[r][k] = win ? g.W[(size_t)(n0 + r) * g.K + k0 + k] : 0.f;
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < KC; ++kk) {
            double m[2], r[2], w[2], wa[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const double xl = sl[ty + 16 * i][kk], xu = su[ty + 16 * i][kk];
                m[i] = 0.5 * (xl + xu);
                r[i] = 0.5 * (xu - xl);
                w[i] = sw[tx + 16 * i][kk];
                wa[i] = fabs(w[i]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    am[i][j] += w[j] * m[i];
                    ar[i][j] += wa[j] * r[i];
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = m0 + ty + 16 * i, col = n0 + tx + 16 * j;
            if (row < g.Mb && col < g.N) {
                const float add = g.bias ? g.bias[col] : 0.f;
                g.Dl[(size_t)row * g.N + col] = (float)(am[i][j] - ar[i][j]) + add;
                g.Du[(size_t)row * g.N + col] = (float)(am[i][j] + ar[i][j]) + add;
            }
        }
}

// Constant-term tile `t` of a small problem: 8 x 8 tiles with the reduction split (few rows: short chains matter), or
// 32 x 32 tiles (many rows: fewer workgroups, more reuse).  The host's count (constant_tiles) follows the same rule.
__device__ __forceinline__ bool wide_constant_tiles(const GemmArgs &g) { return (long long)g.Mb * g.N >= (1 << 17); }
__device__ __forceinline__ void constant_tile(const GemmArgs &g, const int t, float *smem) {
    if (wide_constant_tiles(g)) {
        const int tiles_n = (g.N + 31) / 32;
        if (t / tiles_n < (g.Mb + 31) / 32) wide_tile(g, t / tiles_n, t % tiles_n, smem);
    } else {
        const int tiles_n = (g.N + 7) / 8;
        if (t / tiles_n < (g.Mb + 7) / 8) sliced_tile(g, t / tiles_n, t % tiles_n, smem);
    }
}
static long long constant_tiles(long long rows, long long n) {
    return rows * n >= (1 << 17) ? ((rows + 31) / 32) * ((n + 31) / 32) : ((rows + 7) / 8) * ((n + 7) / 8);
}

__global__ void __launch_bounds__(256) signsplit_gemm_simple(const GemmArgs g) {
    __shared__ float sm[3 * 16 * 17];
    const int tiles_n = (g.N + 15) / 16;
    simple_tile(g, blockIdx.x / tiles_n, blockIdx.x % tiles_n, sm);
}

// Launches the exact-accumulation kernel for the constant-term rows of g (its coefficient rows are left alone).
// (The 8 x 8 tiles with the split reduction, which the small problems take inside their MFMA launch, measured
// 40 - 170 us slower here at 960 rows x 256 .. 512 columns: four times the workgroups re-read W; the 32 x 32 tiles
// that serve many rows there 16 - 70 us slower: a quarter of the workgroups, each a four times longer chain with
// nothing beside it.)
// False if the grid would be too large.
// Few rows (the machine far from full): the 8 x 8 tiles with the split reduction instead -- a 16 x 16 tile alone is a
// chain of K / 16 staged steps (14 us at K = 256), the split one a quarter of that.
__global__ void __launch_bounds__(256) signsplit_gemm_sliced(const GemmArgs g) {
    __shared__ __align__(16) float sm[3 * 8 * 65 + 2 * 4 * 64 * 2];
    const int tiles_n = (g.N + 7) / 8;
    sliced_tile(g, blockIdx.x / tiles_n, blockIdx.x % tiles_n, sm);
}
static bool launch_constant_rows(const GemmArgs &g, hipStream_t st) {
    GemmArgs gb = g;
    gb.Mw = 0;
    if ((long long)g.Mb * g.N <= 64LL * faith::compute_units()) {           // at most one 8 x 8 tile per CU
        const long long grids = ((long long)(g.Mb + 7) / 8) * ((g.N + 7) / 8);
        hipLaunchKernelGGL(signsplit_gemm_sliced, dim3((unsigned)grids), dim3(256), 0, st, gb);
        return true;
    }
    const long long gridb = ((long long)(g.Mb + 15) / 16) * ((g.N + 15) / 16);
    if (gridb > 0x7fffffffLL) return false;
    hipLaunchKernelGGL(signsplit_gemm_simple, dim3((unsigned)gridb), dim3(256), 0, st, gb);
    return true;
}

template <bool EXACT>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
signsplit_gemm(const GemmArgs g, const int b_tiles) {
    __shared__ float sm[2 * 4 * 2 * 128 * 8];            // two stages of four operands, 64 KB
    // the constant-term rows as leading workgroups (b_tiles of them, a multiple of 8): chains of short dependent
    // steps that run beside the MFMA tiles instead of in a launch of their own behind them
    if ((int)blockIdx.x < b_tiles) {
        constant_tile(g, blockIdx.x, sm);
        return;
    }
    signsplit_gemm_body<EXACT, 2, 2>(g, sm, blockIdx.x - b_tiles);
}
// Small problems: the first `b_tiles` workgroups take the 8 x 8 tiles of the constant-term rows
// (exact accumulation; chains of short dependent steps, so they start first and run beside the
// MFMA tiles instead of in a launch of their own), the others one MFMA tile of 64 MBM x 64 MBN each.
template <bool EXACT, int MBM, int MBN>
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_small(const GemmArgs g, const int b_tiles) {
    __shared__ __align__(16) float sm[2 * 4 * 64 * 8 * (MBM + MBN)];   // 32 KB (64 x 64) or 48 KB
    if ((int)blockIdx.x < b_tiles) {
        constant_tile(g, blockIdx.x, sm);
        return;
    }
    signsplit_gemm_body<EXACT, MBM, MBN>(g, sm, blockIdx.x - b_tiles);
}


// Tiny problems (a pooler, a classifier: fewer 64 x 64 tiles than a quarter of the CUs): a 64 x 64 tile is
// one wavefront's chain of K / 2 * 4 MFMAs per 32 x 32 block -- 14 us at K = 256 with nine tenths of the
// machine idle.  Here a workgroup owns ONE 32 x 32 block of C_l and C_u and its four wavefronts split the
// reduction four ways; every wavefront loads its fragments straight from global memory in MFMA layout (lane
// (i, h) holds k = 8 s + 4 h .. + 3 of row i: the same K pairing as the LDS fragments above), so there is
// no staging and no barrier in the loop; the four partial blocks meet in LDS and are added in a fixed
// order.  K % 32 == 0.  The first `b_tiles` workgroups take the constant-term rows, as above.
// `block`: the workgroup's number within its problem; sm: 32 KB ([wavefront][l, u][register][lane]).
__device__ __forceinline__ void ksplit_body(const GemmArgs &g, const int b_tiles, const int block, float *sm) {
    if (block < b_tiles) {
        const int tiles_n = (g.N + 7) / 8;
        const int m_blk = block / tiles_n;
        if (m_blk < (g.Mb + 7) / 8) sliced_tile(g, m_blk, block % tiles_n, sm);
        return;
    }
    constexpr int CH = 4;                                        // K-steps of 8 fetched ahead
    const int pid = block - b_tiles;
    const int tiles_n = (g.N + 31) / 32;
    const int m0 = (pid / tiles_n) * 32, n0 = (pid % tiles_n) * 32;
    const int lane = threadIdx.x % 64, wv = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const int fi = lane % 32, fh = lane / 32;
    const int K = g.K, kw = K / 4, ns = kw / 8;
    // rows past the end re-read the last row; their results are never stored
    const size_t oa = (size_t)min(m0 + fi, g.Mw - 1) * K + wv * kw + 4 * fh;
    const size_t ow = (size_t)min(n0 + fi, g.N - 1) * K + wv * kw + 4 * fh;
    const float4 *__restrict__ pal = reinterpret_cast<const float4 *>(g.Al + oa);
    const float4 *__restrict__ pau = reinterpret_cast<const float4 *>(g.Au + oa);
    const float4 *__restrict__ pw = reinterpret_cast<const float4 *>(g.W + ow);

    floatx16 cl, cu;
#pragma unroll
    for (int r = 0; r < 16; ++r) cl[r] = cu[r] = 0.f;
    float4 al[CH], au[CH], w[CH], nal[CH], nau[CH], nw[CH];
    auto fetch = [&](float4 (&a)[CH], float4 (&b)[CH], float4 (&c)[CH], int s0) {
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if (s0 + i < ns) {
                a[i] = pal[2 * (s0 + i)];
                b[i] = pau[2 * (s0 + i)];
                c[i] = pw[2 * (s0 + i)];
            }
        }
    };
    fetch(al, au, w, 0);
    for (int s0 = 0; s0 < ns; s0 += CH) {
        if (s0 + CH < ns) fetch(nal, nau, nw, s0 + CH);
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            if (s0 + i < ns) {
                // centre / radius form, with ordinary float code: these values feed the MFMAs directly
                const float4 am = mid4(al[i], au[i]), ar = rad4(al[i], au[i]), wa = abs4(w[i]);
#define FAITH_STEP(c)                       \
    cl = mfma(am.c, w[i].c, cl);            \
    cu = mfma(ar.c, wa.c, cu);
                FAITH_STEP(x)
                FAITH_STEP(y)
                FAITH_STEP(z)
                FAITH_STEP(w)
#undef FAITH_STEP
            }
        }
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            al[i] = nal[i];
            au[i] = nau[i];
            w[i] = nw[i];
        }
    }

    // the four partial blocks, added in the order of their K ranges; wavefront v finishes registers 4 v .. 4 v + 3
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        sm[((wv * 2 + 0) * 16 + r) * 64 + lane] = cl[r];
        sm[((wv * 2 + 1) * 16 + r) * 64 + lane] = cu[r];
    }
    __syncthreads();
    const int col = n0 + fi;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int r = 4 * wv + q;
        float sl = sm[((0 * 2 + 0) * 16 + r) * 64 + lane], su = sm[((0 * 2 + 1) * 16 + r) * 64 + lane];
#pragma unroll
        for (int v = 1; v < 4; ++v) {
            sl += sm[((v * 2 + 0) * 16 + r) * 64 + lane];
            su += sm[((v * 2 + 1) * 16 + r) * 64 + lane];
        }
        // register r of a 32 x 32 block is row 8 * (r / 4) + 4 * (lane / 32) + r % 4, column lane % 32;
        // sl is the centre term, su the radius term
        const int row = m0 + 8 * wv + 4 * fh + q;
        if (row < g.Mw && col < g.N) {
            g.Cl[(size_t)row * g.N + col] = 0.5f * (sl - su);
            g.Cu[(size_t)row * g.N + col] = 0.5f * (sl + su);
        }
    }
}
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_ksplit(const GemmArgs g, const int b_tiles) {
    __shared__ __align__(16) float sm[4 * 2 * 16 * 64];
    ksplit_body(g, b_tiles, blockIdx.x, sm);
}


// Up to three GEMMs that share their left operand (the query, key and value layers of an attention block:
// same bound object, three weight matrices of one shape) in ONE launch of the small-tile kernel: at 8192 rows
// a launch is a single round of tiles, and three launches pay the fill and the drain of the machine three times.
struct GroupArgs {
    GemmArgs g;                 // group 0, and the operand shared by all
    const float *W[2], *bias[2];
    float *Cl[2], *Cu[2], *Dl[2], *Du[2];   // groups 1 and 2
    int groups;
};
__device__ __forceinline__ GemmArgs group_of(const GroupArgs &G, const int grp) {
    GemmArgs h = G.g;
    if (grp > 0) {
        const int i = grp - 1;
        h.W = G.W[i];  h.bias = G.bias[i];
        h.Cl = G.Cl[i];  h.Cu = G.Cu[i];  h.Dl = G.Dl[i];  h.Du = G.Du[i];
    }
    return h;
}
// Tiny problems that share their operand (the query, key and value layers on the coefficient rows of one perturbed
// position): `per` workgroups of signsplit_gemm_ksplit per group, one launch.
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_ksplit_grouped(const GroupArgs G, const int b_tiles, const int per) {
    __shared__ __align__(16) float sm[4 * 2 * 16 * 64];
    const GemmArgs h = group_of(G, blockIdx.x / per);
    ksplit_body(h, b_tiles, blockIdx.x % per, sm);
}
// b_tiles constant-term tiles per group first (all groups), then `w_tiles` MFMA tiles per group; both are
// multiples of 8, so a tile keeps the XCD its number within the group gives it.
template <bool EXACT, int MBM, int MBN>
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_grouped(const GroupArgs G, const int b_tiles, const int w_tiles) {
    __shared__ __align__(16) float sm[2 * 4 * 64 * 8 * (MBM + MBN)];
    int pid = blockIdx.x;
    if (pid < b_tiles * G.groups) {
        const GemmArgs h = group_of(G, pid / b_tiles);
        constant_tile(h, pid % b_tiles, sm);
        return;
    }
    pid -= b_tiles * G.groups;
    const GemmArgs h = group_of(G, pid / w_tiles);
    signsplit_gemm_body<EXACT, MBM, MBN>(h, sm, pid % w_tiles);
}

}  // namespace

// Macro-tile of the MFMA kernel for a problem of mw coefficient rows, from tuner runs on 1024 ... 245760 rows, K and
// N 64 ... 1024 (the built-in choice is within 3 % of the best of the four there).  The tuning knob forces a shape.
static void choose_tile(long long mw, int dim_out, int dim_y_out, int *tm, int *tn) {
    auto tiles = [&](int m, int n) { return ((mw + m - 1) / m) * ((dim_y_out + n - 1) / n); };
    const long long cus = faith::compute_units();
    // tiny problems want the most workgroups (64 x 64); up to two 128 x 64 tiles per CU that shape is up to 17 %
    // ahead; 128 x 128 (the most MFMAs per staged operand) pays once there are a dozen of its tiles per CU, whatever
    // the reduction length: 2 - 5 % at 131072 ... 245760 rows with K and N of 256 ... 768 (the batched propagation of
    // a sentence's positions), level at 8 tiles per CU, behind below that, where the pro- and epilogues of five
    // small co-resident workgroups overlap better than those of two large ones
    // (fewer 128 x 64 tiles than CUs would each run alone, one wavefront per SIMD: twice as many 64 x 64 tiles,
    // two on a CU, finish in the time of one -- 2560 rows, K = N = 768: 118 -> 75 us, K = 3072: 451 -> 251 us)
    if (tiles(64, 64) <= cus || tiles(128, 64) < cus) { *tm = 64; *tn = 64; }
    else if (tiles(128, 64) <= 2 * cus) { *tm = 128; *tn = 64; }
    else if (tiles(128, 128) >= 12 * cus) { *tm = 128; *tn = 128; }
    // many column tiles re-read every block of rows from L2: the large tile halves that (3 - 5 % at
    // 768 -> 3072 and 512 -> 2048 with 12288 ... 24576 rows) once it fills the machine four times over
    else if (dim_y_out >= 2048 && tiles(128, 128) >= 8 * cus) { *tm = 128; *tn = 128; }
    else { *tm = 64; *tn = 64; }
    switch (faith::tune_get(FAITH_TUNE_GEMM_VARIANT)) {
        case 1: *tm = 64;  *tn = 64;  break;
        case 2: *tm = 128; *tn = 128; break;
        case 3: *tm = 128; *tn = 64;  break;
        case 4: *tm = 64;  *tn = 128; break;
        default: break;
    }
}

// The layer on mw coefficient rows and `rows` constant-term rows (an ordinary bound object has mw = rows * dim_in).
static int matmul_rows(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw, const float *W,
                       const float *bias, float *y_lb, float *y_ub, float *y_lw, float *y_uw, long long mw, long long rows,
                       int dim_out, int dim_y_out, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(W); FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub);
    if (mw != 0) { FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw); }
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(W);
    FAITH_ALIGNED4(bias); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_REQUIRE(mw >= 0 && rows > 0 && dim_out > 0 && dim_y_out > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_verification: coefficient rows=%lld (>= 0) constant rows=%lld dim_out=%d dim_y_out=%d must be positive",
                  mw, rows, dim_out, dim_y_out);
    FAITH_REQUIRE(mw <= 0x7fffffffLL && rows <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "faith_matmul_verification: batch*length*dim_in exceeds 2^31");
    GemmArgs g{x_lw, x_uw, x_lb, x_ub, W, bias, y_lw, y_uw, y_lb, y_ub, (int)mw, (int)rows, dim_y_out, dim_out};
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (mw == 0) {          // the constant-term rows alone (a caller that multiplies the coefficient rows elsewhere)
        FAITH_REQUIRE(launch_constant_rows(g, st), FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        return faith::check_launch("faith_matmul_verification");
    }
    const bool fast = (dim_out % 4 == 0) && faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) &&
                      faith::aligned(W, 16) && 128LL * dim_out * 4 < 0xffffffffLL &&  // 32-bit offsets in a tile
                      128LL * dim_y_out * 4 < 0x80000000LL;                           // and in a tile of the result
    if (fast) {
        // coefficient rows on MFMA, constant-term rows on the exact-accumulation kernel
        auto tiles = [&](int m, int n) { return ((mw + m - 1) / m) * ((dim_y_out + n - 1) / n); };
        const long long cus = faith::compute_units();
        int tm, tn;
        choose_tile(mw, dim_out, dim_y_out, &tm, &tn);
        const int pick = faith::tune_get(FAITH_TUNE_GEMM_VARIANT);
        // tiny problems with a reduction worth splitting: a 32 x 32 block per workgroup, K over its wavefronts
        if (dim_out % 32 == 0 && (pick == 5 || (pick == 0 && dim_out >= 128 && 4 * tiles(64, 64) <= cus))) {
            const long long gridb = ((rows + 7) / 8) * ((dim_y_out + 7) / 8);
            const long long grid = ((mw + 31) / 32) * ((dim_y_out + 31) / 32);
            FAITH_REQUIRE(grid + gridb <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
            hipLaunchKernelGGL(signsplit_gemm_ksplit, dim3((unsigned)(grid + gridb)), dim3(NTHREADS), 0, st, g, (int)gridb);
            return faith::check_launch("faith_matmul_verification");
        }
        const long long mblks = (mw + tm - 1) / tm;
        const long long grid = ((mblks + XCDS - 1) / XCDS) * XCDS * ((dim_y_out + tn - 1) / tn);
        FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        const bool exact = dim_out % BK == 0;
        if (tm == 128 && tn == 128) {
            const long long b_tiles = (constant_tiles(rows, dim_y_out) + XCDS - 1) / XCDS * XCDS;
            FAITH_REQUIRE(grid + b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
            const dim3 gd((unsigned)(grid + b_tiles));
            if (exact)
                hipLaunchKernelGGL(signsplit_gemm<true>, gd, dim3(NTHREADS), 0, st, g, (int)b_tiles);
            else
                hipLaunchKernelGGL(signsplit_gemm<false>, gd, dim3(NTHREADS), 0, st, g, (int)b_tiles);
        } else {
            // constant-term tiles in front, rounded up to a multiple of 8 so that the MFMA tiles keep
            // their XCD (workgroup number mod 8)
            const long long gridb = constant_tiles(rows, dim_y_out);
            const long long b_tiles = (gridb + XCDS - 1) / XCDS * XCDS;
            FAITH_REQUIRE(grid + b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
            const dim3 gd((unsigned)(grid + b_tiles)), bd(NTHREADS);
#define FAITH_LAUNCH_SMALL(MBM, MBN)                                                                      \
    if (exact) hipLaunchKernelGGL((signsplit_gemm_small<true, MBM, MBN>), gd, bd, 0, st, g, (int)b_tiles); \
    else hipLaunchKernelGGL((signsplit_gemm_small<false, MBM, MBN>), gd, bd, 0, st, g, (int)b_tiles)
            if (tm == 64 && tn == 64) { FAITH_LAUNCH_SMALL(1, 1); }
            else if (tm == 128) { FAITH_LAUNCH_SMALL(2, 1); }
            else { FAITH_LAUNCH_SMALL(1, 2); }
#undef FAITH_LAUNCH_SMALL
        }
    } else {
        const long long grid = ((mw + 15) / 16 + (rows + 15) / 16) * ((dim_y_out + 15) / 16);
        FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        hipLaunchKernelGGL(signsplit_gemm_simple, dim3((unsigned)grid), dim3(256), 0, st, g);
    }
    return faith::check_launch("faith_matmul_verification");
}

extern "C" int faith_matmul_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                         const float *W, const float *bias, float *y_lb, float *y_ub, float *y_lw,
                                         float *y_uw, int batch_size, int length, int dim_in, int dim_out,
                                         int dim_y_out, void *stream) {
    FAITH_REQUIRE(batch_size > 0 && length > 0 && dim_in > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_verification: batch=%d length=%d dim_in=%d must be positive", batch_size, length, dim_in);
    const long long rows = (long long)batch_size * length;
    return matmul_rows(x_lb, x_ub, x_lw, x_uw, W, bias, y_lb, y_ub, y_lw, y_uw, rows * dim_in, rows, dim_out, dim_y_out, stream);
}

extern "C" int faith_matmul_rows_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                              const float *W, const float *bias, float *y_lb, float *y_ub, float *y_lw,
                                              float *y_uw, long long rows_w, long long rows_b, int dim_out, int dim_y_out,
                                              void *stream) {
    return matmul_rows(x_lb, x_ub, x_lw, x_uw, W, bias, y_lb, y_ub, y_lw, y_uw, rows_w, rows_b, dim_out, dim_y_out, stream);
}

static int matmul_group_rows(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw, int groups,
                             const float *const *W, const float *const *bias, float *const *y_lb, float *const *y_ub,
                             float *const *y_lw, float *const *y_uw, long long mw, long long rows, int dim_out, int dim_y_out,
                             void *stream);

extern "C" int faith_matmul_group_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                               int groups, const float *const *W, const float *const *bias,
                                               float *const *y_lb, float *const *y_ub, float *const *y_lw,
                                               float *const *y_uw, int batch_size, int length, int dim_in, int dim_out,
                                               int dim_y_out, void *stream) {
    FAITH_REQUIRE(batch_size > 0 && length > 0 && dim_in > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_group_verification: batch=%d length=%d dim_in=%d must be positive", batch_size, length, dim_in);
    const long long rows = (long long)batch_size * length;
    return matmul_group_rows(x_lb, x_ub, x_lw, x_uw, groups, W, bias, y_lb, y_ub, y_lw, y_uw, rows * dim_in, rows, dim_out,
                             dim_y_out, stream);
}

extern "C" int faith_matmul_group_rows_verification(const float *x_lb, const float *x_ub, const float *x_lw,
                                                    const float *x_uw, int groups, const float *const *W,
                                                    const float *const *bias, float *const *y_lb, float *const *y_ub,
                                                    float *const *y_lw, float *const *y_uw, long long rows_w,
                                                    long long rows_b, int dim_out, int dim_y_out, void *stream) {
    return matmul_group_rows(x_lb, x_ub, x_lw, x_uw, groups, W, bias, y_lb, y_ub, y_lw, y_uw, rows_w, rows_b, dim_out,
                             dim_y_out, stream);
}

static int matmul_group_rows(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw, int groups,
                             const float *const *W, const float *const *bias, float *const *y_lb, float *const *y_ub,
                             float *const *y_lw, float *const *y_uw, long long mw, long long rows, int dim_out, int dim_y_out,
                             void *stream) {
    FAITH_NOT_NULL(W); FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_REQUIRE(groups >= 1 && groups <= 3, FAITH_ERR_SHAPE, "faith_matmul_group_verification: groups=%d must be 1, 2 or 3",
                  groups);
    const long long cus = faith::compute_units();
    auto tiles = [&](int m, int n) { return ((mw + m - 1) / m) * (((long long)dim_y_out + n - 1) / n) * groups; };
    bool fast = mw > 0 && rows > 0 && dim_out > 0 && dim_y_out > 0 && mw <= 0x7fffffffLL && rows <= 0x7fffffffLL &&
                groups > 1 && dim_out % 4 == 0 && x_lb && x_ub && x_lw && x_uw && faith::aligned(x_lb, 4) && faith::aligned(x_ub, 4) &&
                faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) &&
                128LL * dim_out * 4 < 0xffffffffLL && 128LL * dim_y_out * 4 < 0x80000000LL &&
                faith::tune_get(FAITH_TUNE_GEMM_VARIANT) == 0;
    for (int i = 0; fast && i < groups; ++i)
        fast = W[i] && y_lb[i] && y_ub[i] && y_lw[i] && y_uw[i] && faith::aligned(W[i], 16) && faith::aligned(y_lb[i], 4) &&
               faith::aligned(y_ub[i], 4) && faith::aligned(y_lw[i], 4) && faith::aligned(y_uw[i], 4) &&
               (!bias || faith::aligned(bias[i], 4));
    // one launch where the small tiles are the choice for the three problems taken together and no single
    // one of them is a tiny problem (those have a kernel of their own); otherwise one launch each
    int tm = 0, tn = 0;
    if (fast && dim_out % 32 == 0 && dim_out >= 128 && 4 * tiles(64, 64) / groups <= cus) {
        // tiny problems: the kernel that splits the reduction over a workgroup's wavefronts, all groups in one launch
        GroupArgs G{};
        G.g = GemmArgs{x_lw, x_uw, x_lb, x_ub, W[0], bias ? bias[0] : nullptr, y_lw[0], y_uw[0], y_lb[0], y_ub[0], (int)mw, (int)rows,
                       dim_y_out, dim_out};
        for (int i = 1; i < groups; ++i) {
            G.W[i - 1] = W[i];  G.bias[i - 1] = bias ? bias[i] : nullptr;
            G.Cl[i - 1] = y_lw[i];  G.Cu[i - 1] = y_uw[i];  G.Dl[i - 1] = y_lb[i];  G.Du[i - 1] = y_ub[i];
        }
        G.groups = groups;
        const long long gridb = ((rows + 7) / 8) * ((dim_y_out + 7) / 8);
        const long long per = gridb + ((mw + 31) / 32) * ((dim_y_out + 31) / 32);
        FAITH_REQUIRE(per * groups <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_group_verification: grid too large");
        hipLaunchKernelGGL(signsplit_gemm_ksplit_grouped, dim3((unsigned)(per * groups)), dim3(NTHREADS), 0,
                           static_cast<hipStream_t>(stream), G, (int)gridb, (int)per);
        return faith::check_launch("faith_matmul_group_verification");
    }
    if (fast) {
        if (tiles(64, 64) <= cus) { tm = 64; tn = 64; }
        else if (tiles(128, 64) <= 2 * cus) { tm = 128; tn = 64; }
        else if (tiles(128, 128) < 8 * cus) { tm = 64; tn = 64; }
        if (tm == 0) fast = false;
    }
    if (!fast) {
        for (int i = 0; i < groups; ++i) {
            const int rc = matmul_rows(x_lb, x_ub, x_lw, x_uw, W[i], bias ? bias[i] : nullptr, y_lb[i], y_ub[i], y_lw[i], y_uw[i],
                                       mw, rows, dim_out, dim_y_out, stream);
            if (rc != FAITH_OK) return rc;
        }
        return FAITH_OK;
    }
    GroupArgs G{};
    G.g = GemmArgs{x_lw, x_uw, x_lb, x_ub, W[0], bias ? bias[0] : nullptr, y_lw[0], y_uw[0], y_lb[0], y_ub[0], (int)mw, (int)rows,
                   dim_y_out, dim_out};
    for (int i = 1; i < groups; ++i) {
        G.W[i - 1] = W[i];  G.bias[i - 1] = bias ? bias[i] : nullptr;
        G.Cl[i - 1] = y_lw[i];  G.Cu[i - 1] = y_uw[i];  G.Dl[i - 1] = y_lb[i];  G.Du[i - 1] = y_ub[i];
    }
    G.groups = groups;
    const long long mblks = (mw + tm - 1) / tm;
    const long long w_tiles = ((mblks + XCDS - 1) / XCDS) * XCDS * ((dim_y_out + tn - 1) / tn);
    const long long gridb = constant_tiles(rows, dim_y_out);
    const long long b_tiles = (gridb + XCDS - 1) / XCDS * XCDS;
    FAITH_REQUIRE((w_tiles + b_tiles) * groups <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_group_verification: grid too large");
    const dim3 gd((unsigned)((w_tiles + b_tiles) * groups)), bd(NTHREADS);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool exact = dim_out % BK == 0;
#define FAITH_LAUNCH_GROUPED(MBM, MBN)                                                                                 \
    if (exact) hipLaunchKernelGGL((signsplit_gemm_grouped<true, MBM, MBN>), gd, bd, 0, st, G, (int)b_tiles, (int)w_tiles); \
    else hipLaunchKernelGGL((signsplit_gemm_grouped<false, MBM, MBN>), gd, bd, 0, st, G, (int)b_tiles, (int)w_tiles)
    if (tm == 64) { FAITH_LAUNCH_GROUPED(1, 1); }
    else { FAITH_LAUNCH_GROUPED(2, 1); }
#undef FAITH_LAUNCH_GROUPED
    return faith::check_launch("faith_matmul_group_verification");
}


// ------------------------------------------------------------------------------------------------------------
// Affine layer and concretization of its result in ONE launch, for problems of a single round of tiles
// (the reference's 16-position, 64-coordinate case; the classifier at the end of the verifier, whose result
// is concretized at once: VerifierForward.py:300-314).  There the layer and the dual norm are two launches
// of a few microseconds each, and the second only re-reads what the first has just written.
//
// A workgroup owns one position (row) and 32 columns of the result: every coefficient row of that position
// passes through it, so the dual norms over dim_in are complete inside the workgroup.  Wavefront v takes
// the 32-row blocks v, v + 4, ... of the position's dim_in rows, each as one 32 x 32 MFMA block over the whole
// reduction with fragments loaded straight from global memory (the K pairing of signsplit_gemm_ksplit), stores
// the block and folds its column norms into its own slots in LDS; the constant-term row is accumulated in
// double by all threads first (the arithmetic of sliced_tile).  dim_in % (32 words) == 0, K % 8 == 0.
namespace {

struct FusedArgs {
    GemmArgs g;
    float *l, *u;               // [Mb, N] concrete interval of the result
    int D, words;
    float eps, qv;
};

// Layer and dual norm of LARGE problems.  The separate concretize re-reads the 2 * rows * dim_in * N floats the
// layer has just written (1.07 GB, 176 us after configuration 2).  Instead a workgroup here takes the dim_in / BM
// tiles of ONE position and one block of columns in turn, so that the column norms of C_l and C_u over all dim_in
// rows are complete inside the workgroup: each tile's epilogue folds its accumulators into one running value per
// lane and column block (128 more vector-ALU instructions per 64 x 64 wavefront tile), the lane halves and the two
// wavefronts that share a column meet in LDS at the end, and the workgroup writes l and u itself -- from the
// constant terms, which the exact-accumulation kernel has produced in the launch before.  No scratch, a fixed
// order of additions.  One perturbed word, dim_in % BM == 0, K % 16 == 0.
struct NormArgs {
    float *l, *u;      // [Mb, N]
    int D;
    float eps, qv;
};

template <int Q, int MBM, int MBN>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
signsplit_gemm_norms(const GemmArgs g, const NormArgs n) {
    constexpr int BM = 64 * MBM, BN = 64 * MBN;
    __shared__ __align__(16) float sm[2 * 4 * 64 * 8 * (MBM + MBN)];
    const int tiles_n = (g.N + BN - 1) / BN;
    const int xcd = blockIdx.x % XCDS, local = blockIdx.x / XCDS;
    const int pos = (local / tiles_n) * XCDS + xcd;          // the column blocks of a position meet in one L2
    const int n_blk = local % tiles_n;
    if (pos >= g.Mb) return;
    const int per = n.D / BM;
    float pl[MBN], pu[MBN];
#pragma unroll
    for (int b = 0; b < MBN; ++b) pl[b] = pu[b] = 0.f;
    for (int t = 0; t < per; ++t) {
        signsplit_gemm_tile<true, MBM, MBN, Q>(g, sm, pos * per + t, n_blk, pl, pu, n.qv);
        __syncthreads();          // the next tile's first stage overwrites LDS that a slower wavefront may still read
    }
    const int tid = threadIdx.x, lane = tid % 64, wv = tid / 64;
    const int wm = wv / 2, wn = wv % 2, fi = lane % 32, fh = lane / 32;
#pragma unroll
    for (int b = 0; b < MBN; ++b) {
        pl[b] = ncomb<Q>(pl[b], __shfl_xor(pl[b], 32, 64));
        pu[b] = ncomb<Q>(pu[b], __shfl_xor(pu[b], 32, 64));
        if (fh == 0) {
            const int col = (wn * MBN + b) * 32 + fi;
            sm[(0 * 2 + wm) * BN + col] = pl[b];
            sm[(1 * 2 + wm) * BN + col] = pu[b];
        }
    }
    __syncthreads();
    if (tid < BN) {
        const int col = n_blk * BN + tid;
        if (col < g.N) {
            const float nl = ncomb<Q>(sm[(0 * 2 + 0) * BN + tid], sm[(0 * 2 + 1) * BN + tid]);
            const float nu = ncomb<Q>(sm[(1 * 2 + 0) * BN + tid], sm[(1 * 2 + 1) * BN + tid]);
            const size_t o = (size_t)pos * g.N + col;
            // l = lb + (-eps * norm), two roundings as Bounds.concretize has them (Bounds.py:313, 324)
            n.l[o] = __fadd_rn(g.Dl[o], __fmul_rn(-n.eps, nfin<Q>(nl, n.qv)));
            n.u[o] = __fadd_rn(g.Du[o], __fmul_rn(n.eps, nfin<Q>(nu, n.qv)));
        }
    }
}

template <int MBM, int MBN>
void launch_norms(const GemmArgs &g, const NormArgs &n, int q, hipStream_t st) {
    const long long tiles_n = (g.N + 64 * MBN - 1) / (64 * MBN);
    const dim3 gd((unsigned)(((long long)(g.Mb + XCDS - 1) / XCDS) * XCDS * tiles_n)), bd(NTHREADS);
    switch (q) {
        case FAITH_Q_1: hipLaunchKernelGGL((signsplit_gemm_norms<FAITH_Q_1, MBM, MBN>), gd, bd, 0, st, g, n); break;
        case FAITH_Q_2: hipLaunchKernelGGL((signsplit_gemm_norms<FAITH_Q_2, MBM, MBN>), gd, bd, 0, st, g, n); break;
        case FAITH_Q_INF: hipLaunchKernelGGL((signsplit_gemm_norms<FAITH_Q_INF, MBM, MBN>), gd, bd, 0, st, g, n); break;
        default: hipLaunchKernelGGL((signsplit_gemm_norms<Q_GENERAL, MBM, MBN>), gd, bd, 0, st, g, n); break;
    }
}

constexpr int FUSED_MAX_WORDS = 8;

template <int Q>
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_concretize(const FusedArgs f) {
    __shared__ float part[FUSED_MAX_WORDS * 4 * 2 * 64];          // [word][wavefront][l, u][lane]
    __shared__ double red[2][8][32];                               // constant terms: [l, u][K slice][column]
    const GemmArgs &g = f.g;
    const int tiles_n = (g.N + 31) / 32;
    const int row = blockIdx.x / tiles_n, n0 = (blockIdx.x % tiles_n) * 32;
    const int tid = threadIdx.x, lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int K = g.K;

    // ---- constant terms of (row, n0 .. n0 + 31): eight K slices per column, lanes along K
    {
        const int c = tid / 8, ks = tid % 8;
        const float *__restrict__ w = g.W + (size_t)min(n0 + c, g.N - 1) * K;
        const float *__restrict__ xl = g.Bl + (size_t)row * K, *__restrict__ xu = g.Bu + (size_t)row * K;
        double accm = 0.0, accr = 0.0;
        for (int k = ks; k < K; k += 8) {
            const double wk = w[k], a = xl[k], b = xu[k];
            accm += wk * (0.5 * (a + b));
            accr += fabs(wk) * (0.5 * (b - a));
        }
        red[0][ks][c] = accm - accr;
        red[1][ks][c] = accm + accr;
    }
    for (int w = 0; w < f.words; ++w) {
        part[((w * 4 + wv) * 2 + 0) * 64 + lane] = 0.f;
        part[((w * 4 + wv) * 2 + 1) * 64 + lane] = 0.f;
    }

    // ---- coefficient rows: 32 x 32 blocks of this position, one per wavefront at a time
    const int fi = lane % 32, fh = lane / 32;
    const int ns = K / 8, blk = f.D / f.words;
    const float4 *__restrict__ pw = reinterpret_cast<const float4 *>(g.W + (size_t)min(n0 + fi, g.N - 1) * K + 4 * fh);
    const int col = n0 + fi;
    for (int db = wv; db < f.D / 32; db += 4) {
        const size_t r0 = (size_t)row * f.D + db * 32;
        const float4 *__restrict__ pal = reinterpret_cast<const float4 *>(g.Al + (r0 + fi) * K + 4 * fh);
        const float4 *__restrict__ pau = reinterpret_cast<const float4 *>(g.Au + (r0 + fi) * K + 4 * fh);
        floatx16 cl, cu;
#pragma unroll
        for (int r = 0; r < 16; ++r) cl[r] = cu[r] = 0.f;
        constexpr int CH = 4;                                       // K-steps of 8 fetched ahead
        float4 al[CH], au[CH], w[CH], nal[CH], nau[CH], nw[CH];
        auto fetch = [&](float4 (&a)[CH], float4 (&b)[CH], float4 (&c)[CH], int s0) {
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if (s0 + i < ns) {
                    a[i] = pal[2 * (s0 + i)];
                    b[i] = pau[2 * (s0 + i)];
                    c[i] = pw[2 * (s0 + i)];
                }
            }
        };
        fetch(al, au, w, 0);
        for (int s0 = 0; s0 < ns; s0 += CH) {
            if (s0 + CH < ns) fetch(nal, nau, nw, s0 + CH);
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                if (s0 + i < ns) {
                    const float4 am = mid4(al[i], au[i]), ar = rad4(al[i], au[i]), wa = abs4(w[i]);
#define FAITH_STEP(c)                       \
    cl = mfma(am.c, w[i].c, cl);            \
    cu = mfma(ar.c, wa.c, cu);
                    FAITH_STEP(x)
                    FAITH_STEP(y)
                    FAITH_STEP(z)
                    FAITH_STEP(w)
#undef FAITH_STEP
                }
            }
#pragma unroll
            for (int i = 0; i < CH; ++i) {
                al[i] = nal[i];
                au[i] = nau[i];
                w[i] = nw[i];
            }
        }
        // register r of the block is row 8 * (r / 4) + 4 * (lane / 32) + r % 4, column lane % 32
        float pl = 0.f, pu = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float c = cl[r], rd = cu[r];                      // twice the centre and radius terms
            cl[r] = 0.5f * (c - rd);
            cu[r] = 0.5f * (c + rd);
            pl = nacc<Q>(pl, cl[r], f.qv);
            pu = nacc<Q>(pu, cu[r], f.qv);
            if (col < g.N) {
                const size_t o = (r0 + 8 * (r / 4) + 4 * fh + r % 4) * g.N + col;
                g.Cl[o] = cl[r];
                g.Cu[o] = cu[r];
            }
        }
        pl = ncomb<Q>(pl, __shfl_xor(pl, 32, 64));
        pu = ncomb<Q>(pu, __shfl_xor(pu, 32, 64));
        const int w_id = (db * 32) / blk;                           // a block lies inside one perturbed word
        float *slot = part + ((w_id * 4 + wv) * 2) * 64 + lane;
        slot[0] = ncomb<Q>(slot[0], pl);
        slot[64] = ncomb<Q>(slot[64], pu);
    }
    __syncthreads();

    // ---- constant terms out, and the interval: l = lb' - eps * sum over words of the norm (Bounds.py:311-326)
    if (tid < 32 && n0 + tid < g.N) {
        double sl = red[0][0][tid], su = red[1][0][tid];
#pragma unroll
        for (int s = 1; s < 8; ++s) {
            sl += red[0][s][tid];
            su += red[1][s][tid];
        }
        const float add = g.bias ? g.bias[n0 + tid] : 0.f;         // added to the rounded product (Bounds.py:391-395)
        const float lb = (float)sl + add, ub = (float)su + add;
        const size_t o = (size_t)row * g.N + n0 + tid;
        g.Dl[o] = lb;
        g.Du[o] = ub;
        float l = lb, u = ub;
        for (int w = 0; w < f.words; ++w) {
            float nl = 0.f, nu = 0.f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                nl = ncomb<Q>(nl, part[((w * 4 + v) * 2 + 0) * 64 + tid]);
                nu = ncomb<Q>(nu, part[((w * 4 + v) * 2 + 1) * 64 + tid]);
            }
            l = __fadd_rn(l, __fmul_rn(-f.eps, nfin<Q>(nl, f.qv)));
            u = __fadd_rn(u, __fmul_rn(f.eps, nfin<Q>(nu, f.qv)));
        }
        f.l[o] = l;
        f.u[o] = u;
    }
}

// The same launch for SHORT reductions (K = 16 * NS, NS = 2 / 4 / 8): a workgroup owns one position and 16
// columns, a wavefront takes 16-row blocks of the position as 16 x 16 MFMA blocks (v_mfma_f32_16x16x4_f32: half
// the cycles of a 32 x 32 x 2 step for a quarter of the block), and every fragment of a block -- the whole
// reduction -- is requested before the first MFMA, so that a block costs one memory latency instead of one per
// group of K-steps.  Lane group g = lane / 16 holds k = 4 * NS * g .. 4 * NS * (g + 1) - 1 of its row (A) or
// column (W) as NS float4; MFMA (q, c) multiplies component c of piece q, i.e. the four k values
// {4 NS g + 4 q + c : g = 0 .. 3}.  With dim_in = 64 all four wavefronts have a block (the 32 x 32 form leaves
// two idle) and twice as many workgroups share the problem.
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int Q, int NS>
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_concretize_short(const FusedArgs f) {
    constexpr int K = 16 * NS;
    __shared__ float part[FUSED_MAX_WORDS * 4 * 2 * 16];          // [word][wavefront][l, u][column]
    __shared__ double red[2][16][17];                              // constant terms: [l, u][K slice][column]
    const GemmArgs &g = f.g;
    const int tiles_n = (g.N + 15) / 16;
    const int row = blockIdx.x / tiles_n, n0 = (blockIdx.x % tiles_n) * 16;
    const int tid = threadIdx.x, lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int fi = lane % 16, fg = lane / 16;
    const int col = n0 + fi;

    // ---- every load of the first block and of the constant terms goes out first
    const float4 *__restrict__ pw = reinterpret_cast<const float4 *>(g.W + (size_t)min(col, g.N - 1) * K) + NS * fg;
    float4 w[NS];
#pragma unroll
    for (int q = 0; q < NS; ++q) w[q] = pw[q];
    const int blocks = f.D / 16, blk = f.D / f.words;
    float4 al[NS], au[NS];
    auto fetch = [&](int db) {
        const float4 *__restrict__ pal = reinterpret_cast<const float4 *>(g.Al + ((size_t)row * f.D + db * 16 + fi) * K) + NS * fg;
        const float4 *__restrict__ pau = reinterpret_cast<const float4 *>(g.Au + ((size_t)row * f.D + db * 16 + fi) * K) + NS * fg;
#pragma unroll
        for (int q = 0; q < NS; ++q) {
            al[q] = pal[q];
            au[q] = pau[q];
        }
    };
    if (wv < blocks) fetch(wv);

    // ---- constant terms of (row, n0 .. n0 + 15): sixteen K slices per column, lanes along K
    {
        const int c = tid / 16, ks = tid % 16;
        const float *__restrict__ wr = g.W + (size_t)min(n0 + c, g.N - 1) * K;
        const float *__restrict__ xl = g.Bl + (size_t)row * K, *__restrict__ xu = g.Bu + (size_t)row * K;
        double accm = 0.0, accr = 0.0;
#pragma unroll
        for (int i = 0; i < NS; ++i) {
            const int k = ks + 16 * i;
            const double wk = wr[k], a = xl[k], b = xu[k];
            accm += wk * (0.5 * (a + b));
            accr += fabs(wk) * (0.5 * (b - a));
        }
        red[0][ks][c] = accm - accr;
        red[1][ks][c] = accm + accr;
    }
    if (lane < 32)
        for (int wd = 0; wd < f.words; ++wd) part[((wd * 4 + wv) * 2) * 16 + lane] = 0.f;

    // ---- coefficient rows: 16 x 16 blocks of this position, one per wavefront at a time
    float4 wa[NS];
#pragma unroll
    for (int q = 0; q < NS; ++q) wa[q] = abs4(w[q]);
    for (int db = wv; db < blocks; db += 4) {
        const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
        floatx4 cl = zero, cu = zero;
#pragma unroll
        for (int q = 0; q < NS; ++q) {
            const float4 am = mid4(al[q], au[q]), ar = rad4(al[q], au[q]);
#define FAITH_STEP(c)                                                           \
    cl = __builtin_amdgcn_mfma_f32_16x16x4f32(am.c, w[q].c, cl, 0, 0, 0);       \
    cu = __builtin_amdgcn_mfma_f32_16x16x4f32(ar.c, wa[q].c, cu, 0, 0, 0);
            FAITH_STEP(x)
            FAITH_STEP(y)
            FAITH_STEP(z)
            FAITH_STEP(w)
#undef FAITH_STEP
        }
        if (db + 4 < blocks) fetch(db + 4);                       // in flight while this block is finished
        // register r of the block is row 4 * (lane / 16) + r, column lane % 16
        const size_t r0 = (size_t)row * f.D + db * 16 + 4 * fg;
        float pl = 0.f, pu = 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float c = cl[r], rd = cu[r];                      // twice the centre and radius terms
            const float lo = 0.5f * (c - rd), up = 0.5f * (c + rd);
            pl = nacc<Q>(pl, lo, f.qv);
            pu = nacc<Q>(pu, up, f.qv);
            if (col < g.N) {
                g.Cl[(r0 + r) * g.N + col] = lo;
                g.Cu[(r0 + r) * g.N + col] = up;
            }
        }
        pl = ncomb<Q>(pl, __shfl_xor(pl, 16, 64));
        pu = ncomb<Q>(pu, __shfl_xor(pu, 16, 64));
        pl = ncomb<Q>(pl, __shfl_xor(pl, 32, 64));
        pu = ncomb<Q>(pu, __shfl_xor(pu, 32, 64));
        if (fg == 0) {
            const int w_id = (db * 16) / blk;                       // a block lies inside one perturbed word
            float *slot = part + ((w_id * 4 + wv) * 2) * 16 + fi;
            slot[0] = ncomb<Q>(slot[0], pl);
            slot[16] = ncomb<Q>(slot[16], pu);
        }
    }
    __syncthreads();

    // ---- constant terms out, and the interval: l = lb' - eps * sum over words of the norm (Bounds.py:311-326)
    if (tid < 16 && n0 + tid < g.N) {
        double sl = red[0][0][tid], su = red[1][0][tid];
#pragma unroll
        for (int s = 1; s < 16; ++s) {
            sl += red[0][s][tid];
            su += red[1][s][tid];
        }
        const float add = g.bias ? g.bias[n0 + tid] : 0.f;         // added to the rounded product (Bounds.py:391-395)
        const float lb = (float)sl + add, ub = (float)su + add;
        const size_t o = (size_t)row * g.N + n0 + tid;
        g.Dl[o] = lb;
        g.Du[o] = ub;
        float l = lb, u = ub;
        for (int wd = 0; wd < f.words; ++wd) {
            float nl = 0.f, nu = 0.f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                nl = ncomb<Q>(nl, part[((wd * 4 + v) * 2 + 0) * 16 + tid]);
                nu = ncomb<Q>(nu, part[((wd * 4 + v) * 2 + 1) * 16 + tid]);
            }
            l = __fadd_rn(l, __fmul_rn(-f.eps, nfin<Q>(nl, f.qv)));
            u = __fadd_rn(u, __fmul_rn(f.eps, nfin<Q>(nu, f.qv)));
        }
        f.l[o] = l;
        f.u[o] = u;
    }
}

template <int NS>
void launch_concretize_short(const FusedArgs &f, int q, dim3 gd, hipStream_t st) {
    const dim3 bd(NTHREADS);
    switch (q) {
        case FAITH_Q_1: hipLaunchKernelGGL((signsplit_gemm_concretize_short<FAITH_Q_1, NS>), gd, bd, 0, st, f); break;
        case FAITH_Q_2: hipLaunchKernelGGL((signsplit_gemm_concretize_short<FAITH_Q_2, NS>), gd, bd, 0, st, f); break;
        case FAITH_Q_INF: hipLaunchKernelGGL((signsplit_gemm_concretize_short<FAITH_Q_INF, NS>), gd, bd, 0, st, f); break;
        default: hipLaunchKernelGGL((signsplit_gemm_concretize_short<Q_GENERAL, NS>), gd, bd, 0, st, f); break;
    }
}

}  // namespace

extern "C" int faith_matmul_concretize_verification(const float *x_lb, const float *x_ub, const float *x_lw,
                                                    const float *x_uw, const float *W, const float *bias, float *y_lb,
                                                    float *y_ub, float *y_lw, float *y_uw, float *l, float *u,
                                                    int batch_size, int length, int dim_in, int dim_out, int dim_y_out,
                                                    float epsilon, int q, int words, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(W);
    FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_NOT_NULL(l); FAITH_NOT_NULL(u);
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(W);
    FAITH_ALIGNED4(bias); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_ALIGNED4(l); FAITH_ALIGNED4(u);
    FAITH_REQUIRE(batch_size > 0 && length > 0 && dim_in > 0 && dim_out > 0 && dim_y_out > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_concretize_verification: batch=%d length=%d dim_in=%d dim_out=%d dim_y_out=%d must be "
                  "positive", batch_size, length, dim_in, dim_out, dim_y_out);
    FAITH_REQUIRE(words >= 1 && words <= 16 && dim_in % words == 0, FAITH_ERR_SHAPE,
                  "faith_matmul_concretize_verification: words=%d must be in 1..16 and divide dim_in=%d", words, dim_in);
    FusedArgs f{};
    if (!faith::dual_exponent(q, &f.qv)) {
        faith::set_error("faith_matmul_concretize_verification: q=%d is neither FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF nor "
                         "the bits of an exponent in (1, inf)", q);
        return FAITH_ERR_UNSUPPORTED;
    }
    const long long rows = (long long)batch_size * length;
    const long long mw = rows * dim_in;
    const long long cus = faith::compute_units();
    const long long tiles64 = ((mw + 63) / 64) * ((dim_y_out + 63) / 64);
    const long long grid = rows * ((dim_y_out + 31) / 32);
    const int pick = faith::tune_get(FAITH_TUNE_GEMM_VARIANT);
    const bool fits = dim_out % 8 == 0 && dim_in % (32 * words) == 0 && words <= FUSED_MAX_WORDS &&
                      faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) && faith::aligned(W, 16) &&
                      mw <= 0x7fffffffLL && grid <= 0x7fffffffLL;
    // one round of the smallest MFMA tiles at most: beyond that the tiled kernels' reuse of W and of the rows
    // is worth more than the launch saved; and a wavefront's chain of 32 x 32 blocks (each as long as the reduction)
    // no longer than the launch it saves: measured 17 against 19.5 us per call up to 128, 26 against 24 us at 256
    // and 44 against 24 us for the 256 -> 2 classifier (512), whose few positions leave the tiled kernel more
    // workgroups than this one has
    const long long chain = (long long)((dim_in + 127) / 128) * dim_out;
    if (fits && (pick == 6 || pick == 8 || (pick == 0 && tiles64 <= cus && chain <= 128))) {
        f.g = GemmArgs{x_lw, x_uw, x_lb, x_ub, W, bias, y_lw, y_uw, y_lb, y_ub, (int)mw, (int)rows, dim_y_out, dim_out};
        f.l = l; f.u = u; f.D = dim_in; f.words = words; f.eps = epsilon;
        hipStream_t st = static_cast<hipStream_t>(stream);
        // short reductions: 16 x 16 blocks, 16 columns per workgroup (knob value 8 keeps the 32 x 32 form)
        const long long grid16 = rows * ((dim_y_out + 15) / 16);
        if (pick != 8 && (dim_out == 32 || dim_out == 64 || dim_out == 128) && dim_in % (16 * words) == 0 &&
            grid16 <= 0x7fffffffLL) {
            const dim3 gd16((unsigned)grid16);
            if (dim_out == 32) launch_concretize_short<2>(f, q, gd16, st);
            else if (dim_out == 64) launch_concretize_short<4>(f, q, gd16, st);
            else launch_concretize_short<8>(f, q, gd16, st);
            return faith::check_launch("faith_matmul_concretize_verification");
        }
        const dim3 gd((unsigned)grid), bd(NTHREADS);
        switch (q) {
            case FAITH_Q_1: hipLaunchKernelGGL(signsplit_gemm_concretize<FAITH_Q_1>, gd, bd, 0, st, f); break;
            case FAITH_Q_2: hipLaunchKernelGGL(signsplit_gemm_concretize<FAITH_Q_2>, gd, bd, 0, st, f); break;
            case FAITH_Q_INF: hipLaunchKernelGGL(signsplit_gemm_concretize<FAITH_Q_INF>, gd, bd, 0, st, f); break;
            default: hipLaunchKernelGGL(signsplit_gemm_concretize<Q_GENERAL>, gd, bd, 0, st, f); break;
        }
        return faith::check_launch("faith_matmul_concretize_verification");
    }
    // large problems: the tiled kernel, one position's tiles per workgroup, column norms in its epilogue
    {
        int tm = 0, tn = 0;
        choose_tile(mw, dim_out, dim_y_out, &tm, &tn);
        if (tm == 64) tn = 64;                    // 64 x 128 has no instantiation with norms
        // knob value 7 keeps layer and concretize apart (for measuring one against the other)
        const bool tiled = pick != 7 && words == 1 && tiles64 > cus && dim_out % BK == 0 && dim_in % tm == 0 &&
                           faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) && faith::aligned(W, 16) &&
                           128LL * dim_out * 4 < 0xffffffffLL && 128LL * dim_y_out * 4 < 0x80000000LL &&   // 32-bit offsets in a tile
                           mw <= 0x7fffffffLL && (rows + XCDS) * ((dim_y_out + tn - 1) / tn) <= 0x7fffffffLL;
        if (tiled) {
            hipStream_t st = static_cast<hipStream_t>(stream);
            GemmArgs g{x_lw, x_uw, x_lb, x_ub, W, bias, y_lw, y_uw, y_lb, y_ub, (int)mw, (int)rows, dim_y_out, dim_out};
            // the constant terms first: the coefficient kernel reads them when it writes l and u
            FAITH_REQUIRE(launch_constant_rows(g, st), FAITH_ERR_SHAPE, "faith_matmul_concretize_verification: grid too large");
            const NormArgs na{l, u, dim_in, epsilon, f.qv};
            if (tm == 128 && tn == 128) launch_norms<2, 2>(g, na, q, st);
            else if (tm == 128) launch_norms<2, 1>(g, na, q, st);
            else launch_norms<1, 1>(g, na, q, st);
            return faith::check_launch("faith_matmul_concretize_verification");
        }
    }
    const int rc = faith_matmul_verification(x_lb, x_ub, x_lw, x_uw, W, bias, y_lb, y_ub, y_lw, y_uw, batch_size, length,
                                             dim_in, dim_out, dim_y_out, stream);
    if (rc != FAITH_OK) return rc;
    FAITH_REQUIRE(rows <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_concretize_verification: batch*length exceeds 2^31");
    return faith_concretize(y_lb, y_ub, y_lw, y_uw, l, u, (int)rows, dim_in, dim_y_out, epsilon, q, words,
                            FAITH_LAYOUT_NATURAL, stream);
}


// ------------------------------------------------------------------------------------------------------------
// Affine layer, residual connection and layer normalisation without the variance in one pass over the
// coefficients: `dense(x).add(residual).layer_norm(...)` of every encoder sub-block (VerifierForward.py:166,
// 181-189).  Apart, the layer writes its [rows * dim_in, N] result, and the normalisation reads it, reads the
// residual and writes again: three passes over the largest object of the propagation for two adds and a
// multiply per element.  Here a workgroup owns 64 whole rows of the result (64 x N tile, N = 128 or 256: wavefront
// tile 32 x N / 2, the accumulator count of the 128 x 128 tile), so the row means are complete inside it.
// The reduction runs in the order of the plain kernel: the sum in front of the normalisation has the bits it has
// there, and the results differ from the separate launches by the order of the row sums only.
namespace {

template <bool EXACT, int MBN>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
signsplit_gemm_rownorm(const GemmArgs g, const RowNormArgs n, const int b_tiles) {
    extern __shared__ __align__(16) float dyn_sm[];     // two stages of (2 x 64 + 2 x 64 MBN) rows x 16 floats
    if ((int)blockIdx.x < b_tiles) {                    // the layer's constant-term rows, as in signsplit_gemm
        constant_tile(g, blockIdx.x, dyn_sm);
        return;
    }
    signsplit_gemm_tile<EXACT, 1, MBN, -1, EPI_ROWNORM, RowNormArgs>(g, dyn_sm, blockIdx.x - b_tiles, 0, nullptr, nullptr, 0.f, n);
}

template <bool EXACT, int MBN>
bool launch_rownorm(const GemmArgs &g, const RowNormArgs &n, hipStream_t st) {
    const size_t lds = 2 * 4 * 64 * 8 * (1 + MBN) * sizeof(float);
    if (!faith::reserve_lds(signsplit_gemm_rownorm<EXACT, MBN>, lds)) return false;
    const long long b_tiles = (constant_tiles(g.Mb, g.N) + XCDS - 1) / XCDS * XCDS;
    const long long grid = (g.Mw + 63) / 64 + b_tiles;
    if (grid > 0x7fffffffLL) return false;
    hipLaunchKernelGGL((signsplit_gemm_rownorm<EXACT, MBN>), dim3((unsigned)grid), dim3(NTHREADS), lds, st, g, n, (int)b_tiles);
    return true;
}

}  // namespace

extern "C" int faith_matmul_layer_norm_fits(long long rows, int dim_in, int dim_out, int dim_y_out, int res_words) {
    const bool taken = rows > 0 && dim_in > 0 && dim_out > 0 && dim_out % 4 == 0 && (dim_y_out == 128 || dim_y_out == 256) &&
                       (res_words == 0 || dim_in % 64 == 0) && 64LL * dim_out * 4 < 0xffffffffLL &&
                       rows * dim_in <= 0x7fffffffLL;
    if (!taken) return 0;
    // a 64-row tile runs through the whole reduction for all columns: with fewer than two of them per compute unit
    // the separate launches, whose layer splits the columns over more workgroups, finish first (measured at
    // N = 128 and 256, reductions of 128 .. 512: even at 512 tiles, 15 - 40 % faster at 1024, slower below)
    return (rows * dim_in + 63) / 64 >= 2LL * faith::compute_units() ? 2 : 1;
}

extern "C" int faith_matmul_layer_norm_verification(const float *x_lb, const float *x_ub, const float *x_lw,
                                                    const float *x_uw, const float *W, const float *bias,
                                                    const float *res_lb, const float *res_ub, const float *res_lw,
                                                    const float *res_uw, const long long *res_positions, int res_words,
                                                    const float *weight, const float *norm_bias, float *y_lb, float *y_ub,
                                                    float *y_lw, float *y_uw, int batch_size, int length, int dim_in,
                                                    int dim_out, int dim_y_out, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(W);
    FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(bias); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub);
    FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw); FAITH_ALIGNED4(res_lb); FAITH_ALIGNED4(res_ub); FAITH_ALIGNED4(res_lw);
    FAITH_ALIGNED4(res_uw); FAITH_ALIGNED4(weight); FAITH_ALIGNED4(norm_bias);
    FAITH_REQUIRE(faith::aligned(res_positions, 8), FAITH_ERR_ALIGN, "faith_matmul_layer_norm_verification: res_positions is not 8-byte aligned");
    FAITH_REQUIRE(batch_size > 0 && length > 0 && dim_in > 0 && dim_out > 0 && dim_y_out > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_layer_norm_verification: batch=%d length=%d dim_in=%d dim_out=%d dim_y_out=%d must be "
                  "positive", batch_size, length, dim_in, dim_out, dim_y_out);
    const bool adding = res_lb || res_ub || res_lw || res_uw;
    FAITH_REQUIRE(!adding || (res_lb && res_ub && res_lw && res_uw), FAITH_ERR_NULL,
                  "faith_matmul_layer_norm_verification: the four tensors of the added object must be given together");
    FAITH_REQUIRE(res_words >= 0 && (res_words == 0) == (res_positions == nullptr) && (res_words == 0 || adding),
                  FAITH_ERR_SHAPE, "faith_matmul_layer_norm_verification: res_words=%d and res_positions must be given "
                  "together, with an added object", res_words);
    FAITH_REQUIRE(faith_matmul_layer_norm_fits((long long)batch_size * length, dim_in, dim_out, dim_y_out, res_words) &&
                  faith::aligned(x_lw, 16) &&
                  faith::aligned(x_uw, 16) && faith::aligned(W, 16), FAITH_ERR_UNSUPPORTED,
                  "faith_matmul_layer_norm_verification: dim_y_out=%d must be 128 or 256, dim_out=%d a multiple of 4, "
                  "dim_in=%d a multiple of 64 when the added object holds some positions only, batch*length*dim_in below "
                  "2^31, and x_lw, x_uw, W 16-byte aligned", dim_y_out, dim_out, dim_in);
    const long long rows = (long long)batch_size * length, mw = rows * dim_in;
    hipStream_t st = static_cast<hipStream_t>(stream);
    GemmArgs g{x_lw, x_uw, x_lb, x_ub, W, bias, y_lw, y_uw, y_lb, y_ub, (int)mw, (int)rows, dim_y_out, dim_out};
    const RowNormArgs n{res_lw, res_uw, res_positions, res_words, length, dim_in, weight, y_lw, y_uw};
    const bool exact = dim_out % BK == 0;
    bool ok;
    if (dim_y_out == 256) ok = exact ? launch_rownorm<true, 4>(g, n, st) : launch_rownorm<false, 4>(g, n, st);
    else ok = exact ? launch_rownorm<true, 2>(g, n, st) : launch_rownorm<false, 2>(g, n, st);
    FAITH_REQUIRE(ok, FAITH_ERR_UNSUPPORTED, "faith_matmul_layer_norm_verification: the device refused the LDS size, or the grid is too large");
    // constant terms (exact accumulation, leading workgroups of that launch): the same normalisation on
    // [rows, dim_y_out] in place (a row is held in registers between its read and its write)
    const int rc = faith::check_launch("faith_matmul_layer_norm_verification");
    if (rc != FAITH_OK) return rc;
    return faith_layer_norm_verification(y_lb, y_ub, y_lw, y_uw, res_lb, res_ub, adding ? res_lw : nullptr,
                                         adding ? res_uw : nullptr, weight, norm_bias, y_lb, y_ub, y_lw, y_uw, 0, rows,
                                         dim_y_out, stream);
}


// ------------------------------------------------------------------------------------------------------------
// Affine layer and ReLU relaxation in one pass over the coefficients: `dense(x).relu()` of the feed-forward
// block (VerifierForward.py:171-179 with hidden_act "relu").  Apart, the layer writes its [rows * dim_in, N]
// result and the relaxation reads it, finds each neuron's concrete interval from the column norms over the
// dim_in rows of its position, scales and writes again.  Here a tile holds all dim_in rows of one position
// (dim_in = 128: the 128 x 128 tile; 256: 256 x 64, wavefront tile 128 x 32, the same accumulator count), so the
// norms, the interval and the two slopes are known before the tile is stored.  One perturbed word.
namespace {

template <bool EXACT, int MBM, int MBN, int Q>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
signsplit_gemm_relu(const GemmArgs g, const ReluArgs r, const float qv) {
    extern __shared__ __align__(16) float dyn_sm[];
    constexpr int BN = 64 * MBN;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int xcd = blockIdx.x % XCDS, local = blockIdx.x / XCDS;
    const int pos = (local / tiles_n) * XCDS + xcd;          // the column blocks of a position meet in one L2
    if (pos >= g.Mb) return;
    signsplit_gemm_tile<EXACT, MBM, MBN, Q, EPI_RELU, ReluArgs>(g, dyn_sm, pos, local % tiles_n, nullptr, nullptr, qv, r);
}

template <bool EXACT, int MBM, int MBN>
const void *relu_kernel(int q) {
    switch (q) {
        case FAITH_Q_1: return reinterpret_cast<const void *>(signsplit_gemm_relu<EXACT, MBM, MBN, FAITH_Q_1>);
        case FAITH_Q_2: return reinterpret_cast<const void *>(signsplit_gemm_relu<EXACT, MBM, MBN, FAITH_Q_2>);
        case FAITH_Q_INF: return reinterpret_cast<const void *>(signsplit_gemm_relu<EXACT, MBM, MBN, FAITH_Q_INF>);
        default: return reinterpret_cast<const void *>(signsplit_gemm_relu<EXACT, MBM, MBN, Q_GENERAL>);
    }
}

}  // namespace

extern "C" int faith_matmul_relu_fits(long long rows, int dim_in, int dim_out, int dim_y_out, int words) {
    const bool taken = rows > 0 && rows <= 0x7fffffffLL / 256 && (dim_in == 128 || dim_in == 256) && dim_out > 0 &&
                       dim_out % 4 == 0 && dim_y_out > 0 && words == 1 && 256LL * dim_out * 4 < 0xffffffffLL &&
                       256LL * dim_y_out * 4 < 0x80000000LL;
    if (!taken) return 0;
    // one tile per position and block of columns: as the 128 x 128 tiles of the plain layer, they pay once they fill
    // the device about twice over
    const long long tiles = rows * ((dim_y_out + (dim_in == 128 ? 127 : 63)) / (dim_in == 128 ? 128 : 64));
    return tiles >= 2LL * faith::compute_units() ? 2 : 1;
}

extern "C" int faith_matmul_relu_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                              const float *W, const float *bias, float *y_lb, float *y_ub, float *y_lw,
                                              float *y_uw, int batch_size, int length, int dim_in, int dim_out,
                                              int dim_y_out, float epsilon, int q, int words, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(W);
    FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(bias); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub);
    FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_REQUIRE(batch_size > 0 && length > 0 && dim_in > 0 && dim_out > 0 && dim_y_out > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_relu_verification: batch=%d length=%d dim_in=%d dim_out=%d dim_y_out=%d must be positive",
                  batch_size, length, dim_in, dim_out, dim_y_out);
    float qv = 0.f;
    if (!faith::dual_exponent(q, &qv)) {
        faith::set_error("faith_matmul_relu_verification: q=%d is neither FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF nor the bits "
                         "of an exponent in (1, inf)", q);
        return FAITH_ERR_UNSUPPORTED;
    }
    const long long rows = (long long)batch_size * length;
    FAITH_REQUIRE(faith_matmul_relu_fits(rows, dim_in, dim_out, dim_y_out, words) && faith::aligned(x_lw, 16) &&
                  faith::aligned(x_uw, 16) && faith::aligned(W, 16), FAITH_ERR_UNSUPPORTED,
                  "faith_matmul_relu_verification: dim_in=%d must be 128 or 256, words=%d one, dim_out=%d a multiple of 4, "
                  "and x_lw, x_uw, W 16-byte aligned", dim_in, words, dim_out);
    hipStream_t st = static_cast<hipStream_t>(stream);
    GemmArgs g{x_lw, x_uw, x_lb, x_ub, W, bias, y_lw, y_uw, y_lb, y_ub, (int)(rows * dim_in), (int)rows, dim_y_out, dim_out};
    const bool exact = dim_out % BK == 0, wide = dim_in == 128;      // 128 x 128 tiles, or 256 x 64
    const void *kernel = wide ? (exact ? relu_kernel<true, 2, 2>(q) : relu_kernel<false, 2, 2>(q))
                              : (exact ? relu_kernel<true, 4, 1>(q) : relu_kernel<false, 4, 1>(q));
    const size_t lds = 2 * 4 * 64 * 8 * (wide ? 4 : 5) * sizeof(float);
    const long long tiles_n = (dim_y_out + (wide ? 127 : 63)) / (wide ? 128 : 64);
    const long long grid = ((rows + XCDS - 1) / XCDS) * XCDS * tiles_n;
    const long long gridb = ((rows + 15) / 16) * ((dim_y_out + 15) / 16);
    FAITH_REQUIRE(gridb <= 0x7fffffffLL && grid <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "faith_matmul_relu_verification: grid too large");
    FAITH_REQUIRE(lds <= 64 * 1024 || hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess,
                  FAITH_ERR_UNSUPPORTED, "faith_matmul_relu_verification: the device refused the LDS size");
    // the constant terms of the layer first: the coefficient kernel reads them when it forms the intervals, and
    // writes the constant terms of the relaxed object over them
    launch_constant_rows(g, st);
    ReluArgs r{y_lb, y_ub, epsilon};
    void *args[] = {&g, &r, &qv};
    if (hipLaunchKernel(kernel, dim3((unsigned)grid), dim3(NTHREADS), args, lds, st) != hipSuccess) {
        faith::set_error("faith_matmul_relu_verification: launch failed: %s", hipGetErrorString(hipGetLastError()));
        return FAITH_ERR_LAUNCH;
    }
    return faith::check_launch("faith_matmul_relu_verification");
}

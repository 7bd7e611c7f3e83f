// Sign-split affine bound propagation  y = x @ W^T (+ bias)  on fp32 MFMA.
//
// Arithmetic of the reference's Bounds.ori_matmul + add
// (Transformer_Verification_Code/Verifiers/Bounds.py:397-413, :383-395):
//     C_l = A_l @ W+ + A_u @ W-        C_u = A_u @ W+ + A_l @ W-
// with W+ = max(W, 0), W- = min(W, 0) (value-identical to W*(W>0), W - W+).
// A_l, A_u are the bound rows ([rows*D_in, H] for lw/uw, [rows, H] for lb/ub, both K-contiguous),
// W is [N, H] as nn.Linear stores it, so both operands stream along K.
//
// The MFMA kernel can take the constant-term rows as trailing M-blocks of the same grid (as the
// reference's CUTLASS path does: tvm_kernels/cuda_kernel/mma/mma_kernel.h:251-259), but the entry
// point sends them to the exact-accumulation kernel below instead: they are 1/D_in of the work
// and the only outputs whose O(1) terms cancel.
//
// Tiling (gfx950): workgroup = 4 wavefronts, macro-tile BM x BN = 128 x 128, K-step 16,
// wavefront tile 64 x 64 = 2 x 2 v_mfma_f32_32x32x2_f32 blocks for EACH of C_l and C_u
// (128 accumulator registers).  Every fragment set (A_l, A_u, W+, W-) feeds four MFMAs, so one
// 16-byte LDS read per operand block covers four K-pairs: 6 LDS reads per 64 MFMAs.  W+ / W-
// are formed with v_max / v_min after the LDS read; W itself is staged once, unsplit.
// LDS rows are padded to K-step + 4 floats so that the 16-byte reads of 8 neighbouring lanes
// fall in distinct banks.  Global -> register -> LDS staging is double-buffered: the loads of
// K-step t+1 are in flight while step t is multiplied; one barrier per K-step.
//
// blockIdx -> tile mapping is XCD-aware: workgroups are dealt round-robin to the 8 XCDs, so
// the N-tiles that share an M-block (and with it A_l / A_u rows) are given ids 8 apart and
// meet in the same L2.
#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 16;
constexpr int LDK = BK + 4;          // padded LDS row
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

__device__ __forceinline__ float4 ld4(const float *p) { return *reinterpret_cast<const float4 *>(p); }

__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
signsplit_gemm(const GemmArgs g) {
    __shared__ float sAl[2][BM * LDK];
    __shared__ float sAu[2][BM * LDK];
    __shared__ float sW[2][BN * LDK];

    // ---- tile of this workgroup
    const int tiles_n = (g.N + BN - 1) / BN;
    const int mblk_w = (g.Mw + BM - 1) / BM;
    const int mblk_b = (g.Mb + BM - 1) / BM;
    const int pid = blockIdx.x;
    const int xcd = pid % XCDS, local = pid / XCDS;
    const int m_blk = (local / tiles_n) * XCDS + xcd;
    const int n_blk = local % tiles_n;
    if (m_blk >= mblk_w + mblk_b) return;
    const bool brows = m_blk >= mblk_w;
    const float *__restrict__ Al = brows ? g.Bl : g.Al;
    const float *__restrict__ Au = brows ? g.Bu : g.Au;
    float *__restrict__ Cl = brows ? g.Dl : g.Cl;
    float *__restrict__ Cu = brows ? g.Du : g.Cu;
    const int M = brows ? g.Mb : g.Mw;
    const int m0 = (brows ? m_blk - mblk_w : m_blk) * BM;
    const int n0 = n_blk * BN;
    const int K = g.K;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int wm = wv / 2, wn = wv % 2;            // 2 x 2 wavefronts, 64 x 64 each

    // ---- staging: a tile is 128 rows x 16 floats = 512 float4, two per thread per operand
    const int kq = tid % 4;                        // which float4 of the 16-float row
    const int r0 = tid / 4;                        // rows r0 and r0 + 64
    size_t offA[2], offW[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int ra = min(m0 + r0 + 64 * i, M - 1);       // rows past the end re-read the last row;
        const int rw = min(n0 + r0 + 64 * i, g.N - 1);     // their products are never stored
        offA[i] = (size_t)ra * K + kq * 4;
        offW[i] = (size_t)rw * K + kq * 4;
    }
    float4 pal[2], pau[2], pw[2];
    auto gload = [&](int kt) {
        const int k = kt * BK;
        const bool in = k + kq * 4 < K;            // K % 4 == 0: a float4 is all in or all out
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (in) {
                pal[i] = ld4(Al + offA[i] + k);
                pau[i] = ld4(Au + offA[i] + k);
                pw[i] = ld4(g.W + offW[i] + k);
            } else {
                pal[i] = pau[i] = pw[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    };
    auto lstore = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int o = (r0 + 64 * i) * LDK + kq * 4;
            *reinterpret_cast<float4 *>(&sAl[buf][o]) = pal[i];
            *reinterpret_cast<float4 *>(&sAu[buf][o]) = pau[i];
            *reinterpret_cast<float4 *>(&sW[buf][o]) = pw[i];
        }
    };

    floatx16 cl[2][2], cu[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;

    // fragment addresses: lane (i = lane % 32, h = lane / 32) reads k = 8*ks + 4*h .. +3 of row i
    const int fi = lane % 32, fh = lane / 32;
    const int fa = (wm * 64 + fi) * LDK + fh * 4;
    const int fw = (wn * 64 + fi) * LDK + fh * 4;

    const int nk = (K + BK - 1) / BK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) gload(kt + 1);
#pragma unroll
        for (int ks = 0; ks < BK / 8; ++ks) {
            float4 al[2], au[2], wp[2], wq[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                al[s] = *reinterpret_cast<const float4 *>(&sAl[buf][fa + s * 32 * LDK + ks * 8]);
                au[s] = *reinterpret_cast<const float4 *>(&sAu[buf][fa + s * 32 * LDK + ks * 8]);
                const float4 w = *reinterpret_cast<const float4 *>(&sW[buf][fw + s * 32 * LDK + ks * 8]);
                wp[s] = make_float4(fmaxf(w.x, 0.f), fmaxf(w.y, 0.f), fmaxf(w.z, 0.f), fmaxf(w.w, 0.f));
                wq[s] = make_float4(fminf(w.x, 0.f), fminf(w.y, 0.f), fminf(w.z, 0.f), fminf(w.w, 0.f));
            }
#define FAITH_STEP(c)                                                           \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) _Pragma("unroll") for (int b = 0; b < 2; ++b) { \
        cl[a][b] = mfma(al[a].c, wp[b].c, cl[a][b]);                            \
        cu[a][b] = mfma(au[a].c, wp[b].c, cu[a][b]);                            \
    }                                                                           \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) _Pragma("unroll") for (int b = 0; b < 2; ++b) { \
        cl[a][b] = mfma(au[a].c, wq[b].c, cl[a][b]);                            \
        cu[a][b] = mfma(al[a].c, wq[b].c, cu[a][b]);                            \
    }
            FAITH_STEP(x)
            FAITH_STEP(y)
            FAITH_STEP(z)
            FAITH_STEP(w)
#undef FAITH_STEP
        }
        if (kt + 1 < nk) lstore(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: register r of a 32x32 block is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int col = n0 + wn * 64 + b * 32 + fi;
        if (col >= g.N) continue;
        const float add = (brows && g.bias) ? g.bias[col] : 0.f;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wm * 64 + a * 32 + 8 * (r / 4) + 4 * fh + (r % 4);
                if (row < M) {
                    const size_t o = (size_t)row * g.N + col;
                    __builtin_nontemporal_store(cl[a][b][r] + add, &Cl[o]);
                    __builtin_nontemporal_store(cu[a][b][r] + add, &Cu[o]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------ exact-accumulation kernel
// 16 x 16 outputs per workgroup, scalar loads, products and sums in double (an fp32 x fp32
// product is exact in double), one rounding at the end.  Two uses:
//  * the constant-term rows lb' / ub': 1/D_in of the work, but their terms are O(1) and cancel,
//    which is where the order of an fp32 summation shows; accumulated in double they carry no
//    summation error at all;
//  * any shape the MFMA kernel does not take (K not a multiple of 4, unaligned pointers).
__global__ void __launch_bounds__(256) signsplit_gemm_simple(const GemmArgs g) {
    __shared__ float sl[16][17], su[16][17], sw[16][17];
    const int mblk_w = (g.Mw + 15) / 16;
    const int tiles_n = (g.N + 15) / 16;
    const int m_blk = blockIdx.x / tiles_n, n_blk = blockIdx.x % tiles_n;
    const bool brows = m_blk >= mblk_w;
    const float *Al = brows ? g.Bl : g.Al, *Au = brows ? g.Bu : g.Au;
    float *Cl = brows ? g.Dl : g.Cl, *Cu = brows ? g.Du : g.Cu;
    const int M = brows ? g.Mb : g.Mw;
    const int m0 = (brows ? m_blk - mblk_w : m_blk) * 16, n0 = n_blk * 16;
    const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    double accl = 0.0, accu = 0.0;
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
            const float w = sw[tx][kk];
            const double wp = fmaxf(w, 0.f), wq = fminf(w, 0.f);
            const double xl = sl[ty][kk], xu = su[ty][kk];
            accl += xl * wp + xu * wq;
            accu += xu * wp + xl * wq;
        }
        __syncthreads();
    }
    const int row = m0 + ty, col = n0 + tx;
    if (row < M && col < g.N) {
        // the reference adds the bias to the rounded fp32 product (Bounds.py:391-395)
        const float add = (brows && g.bias) ? g.bias[col] : 0.f;
        Cl[(size_t)row * g.N + col] = (float)accl + add;
        Cu[(size_t)row * g.N + col] = (float)accu + add;
    }
}

}  // namespace

extern "C" int faith_matmul_verification(const float *x_lb, const float *x_ub, const float *x_lw, const float *x_uw,
                                         const float *W, const float *bias, float *y_lb, float *y_ub, float *y_lw,
                                         float *y_uw, int batch_size, int length, int dim_in, int dim_out,
                                         int dim_y_out, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(W);
    FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(W);
    FAITH_ALIGNED4(bias); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_REQUIRE(batch_size > 0 && length > 0 && dim_in > 0 && dim_out > 0 && dim_y_out > 0, FAITH_ERR_SHAPE,
                  "faith_matmul_verification: batch=%d length=%d dim_in=%d dim_out=%d dim_y_out=%d must be positive",
                  batch_size, length, dim_in, dim_out, dim_y_out);
    const long long rows = (long long)batch_size * length;
    const long long mw = rows * dim_in;
    FAITH_REQUIRE(mw <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: batch*length*dim_in exceeds 2^31");
    GemmArgs g{x_lw, x_uw, x_lb, x_ub, W, bias, y_lw, y_uw, y_lb, y_ub, (int)mw, (int)rows, dim_y_out, dim_out};
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool fast = (dim_out % 4 == 0) && faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) &&
                      faith::aligned(x_lb, 16) && faith::aligned(x_ub, 16) && faith::aligned(W, 16);
    if (fast) {
        // coefficient rows on MFMA, constant-term rows on the exact-accumulation kernel
        GemmArgs gw = g;
        gw.Mb = 0;
        const long long mblks = (mw + BM - 1) / BM;
        const long long grid = ((mblks + XCDS - 1) / XCDS) * XCDS * ((dim_y_out + BN - 1) / BN);
        FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        hipLaunchKernelGGL(signsplit_gemm, dim3((unsigned)grid), dim3(NTHREADS), 0, st, gw);
        GemmArgs gb = g;
        gb.Mw = 0;
        const long long gridb = ((rows + 15) / 16) * ((dim_y_out + 15) / 16);
        hipLaunchKernelGGL(signsplit_gemm_simple, dim3((unsigned)gridb), dim3(256), 0, st, gb);
    } else {
        const long long grid = ((mw + 15) / 16 + (rows + 15) / 16) * ((dim_y_out + 15) / 16);
        FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        hipLaunchKernelGGL(signsplit_gemm_simple, dim3((unsigned)grid), dim3(256), 0, st, g);
    }
    return faith::check_launch("faith_matmul_verification");
}

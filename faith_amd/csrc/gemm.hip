// Sign-split affine bound propagation  y = x @ W^T (+ bias)  on fp32 MFMA.
//
// Arithmetic of the reference's Bounds.ori_matmul + add
// (Transformer_Verification_Code/Verifiers/Bounds.py:397-413, :383-395):
//     C_l = A_l @ W+ + A_u @ W-        C_u = A_u @ W+ + A_l @ W-
// with W+ = max(W, 0), W- = min(W, 0) (value-identical to W*(W>0), W - W+).
// A_l, A_u are the bound rows ([rows*D_in, H] for lw/uw, [rows, H] for lb/ub, both K-contiguous),
// W is [N, H] as nn.Linear stores it, so both operands stream along K.
//
// The reference's CUTLASS path takes the constant-term rows as trailing M-blocks of the same grid
// (tvm_kernels/cuda_kernel/mma/mma_kernel.h:251-259); here they go to the exact-accumulation
// code below instead: they are 1/D_in of the work and the only outputs whose O(1) terms cancel.
// For small problems those tiles are the leading workgroups of the MFMA launch, for large ones a
// launch of their own.
//
// Tiling (gfx950): workgroup = 4 wavefronts, macro-tile BM x BN = 128 x 128, K-step 16,
// wavefront tile 64 x 64 = 2 x 2 v_mfma_f32_32x32x2_f32 blocks for EACH of C_l and C_u
// (128 accumulator registers).  Every fragment set (A_l, A_u, W+, W-) feeds four MFMAs, so one
// 16-byte LDS read per operand block covers four K-pairs: 8 LDS reads per 64 MFMAs.
//
// On this part every vector-ALU instruction a wavefront issues takes its slot from the MFMA pipe,
// so the K-loop issues almost none: W is split by sign ONCE, by the thread that stages it (W+ and
// W- are separate LDS tiles); global addresses are buffer addresses (a wave-uniform descriptor and
// K offset, one per-thread offset per row that never changes), and the K-step is straight-line:
// fetch of step t+1, half the MFMAs of step t, staging of step t+1, the other half, one barrier.
//
// LDS: a K-step of an operand is two [128 x 8] halves; rows are 8 floats with the two 16-byte
// pieces swapped on every other group of four rows, which makes the 16-byte stores and the
// 16-byte fragment reads bank-conflict free without padding.  4 operands x 8 KB x 2 stages = 64 KB,
// two workgroups per CU.
//
// blockIdx -> tile mapping is XCD-aware: workgroups are dealt round-robin to the 8 XCDs, so
// the N-tiles that share an M-block (and with it A_l / A_u rows) are given ids 8 apart and
// meet in the same L2.
#include "common.h"

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
// max(v, 0) / min(v, 0) as single instructions (fmaxf / fminf add a canonicalising v_max each)
__device__ __forceinline__ float pos1(float v) {
    float r;
    asm("v_max_f32 %0, 0, %1" : "=v"(r) : "v"(v));
    return r;
}
__device__ __forceinline__ float neg1(float v) {
    float r;
    asm("v_min_f32 %0, 0, %1" : "=v"(r) : "v"(v));
    return r;
}
__device__ __forceinline__ float4 pos4(float4 v) { return make_float4(pos1(v.x), pos1(v.y), pos1(v.z), pos1(v.w)); }
__device__ __forceinline__ float4 neg4(float4 v) { return make_float4(neg1(v.x), neg1(v.y), neg1(v.z), neg1(v.w)); }

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
// MB = MFMA blocks per wavefront and dimension: 2 is the 128 x 128 macro-tile described above; 1 is a
// 64 x 64 macro-tile (wavefront tile 32 x 32, 32 accumulator registers, 32 KB of LDS) for problems
// with too few 128 x 128 tiles to fill the machine: a wavefront then works through 32 MFMAs per
// K-step instead of 128, a quarter of the latency, at a lower MFMA rate per byte staged.
template <bool EXACT, int MB>
__device__ __forceinline__ void signsplit_gemm_body(const GemmArgs &g, float *smem, const int pid) {
    constexpr int BM = 64 * MB, BN = 64 * MB;
    constexpr int HALF = BM * 8;             // floats in one [BM x 8] half of an operand's K-step
    constexpr int OPER = 2 * HALF;           // one operand, one K-step
    constexpr int S_AL = 0, S_AU = OPER, S_WP = 2 * OPER, S_WN = 3 * OPER, STAGE = 4 * OPER;
    float(*sm)[STAGE] = reinterpret_cast<float(*)[STAGE]>(smem);

    // ---- tile of this workgroup
    const int tiles_n = (g.N + BN - 1) / BN;
    const int mblks = (g.Mw + BM - 1) / BM;
    const int xcd = pid % XCDS, local = pid / XCDS;
    const int m_blk = (local / tiles_n) * XCDS + xcd;
    const int n_blk = local % tiles_n;
    if (m_blk >= mblks) return;
    const int M = g.Mw;
    const int m0 = m_blk * BM, n0 = n_blk * BN;
    const int K = g.K;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wm = wv / 2, wn = wv % 2;            // 2 x 2 wavefronts, (32 MB) x (32 MB) each

    // ---- staging: an operand's K-step is BM rows x 16 floats = 256 MB float4, MB per thread:
    // piece kq of rows r0 (and r0 + 64).  Offsets are relative to the first row of the tile (the entry
    // point checks that a tile's rows span less than 4 GB); rows past the end re-read the last row, their
    // products are never stored.
    const int kq = tid % 4, r0 = tid / 4;
    const __amdgpu_buffer_rsrc_t wal = window(g.Al + (size_t)m0 * K, ((size_t)(M - m0) * K) * 4);
    const __amdgpu_buffer_rsrc_t wau = window(g.Au + (size_t)m0 * K, ((size_t)(M - m0) * K) * 4);
    const __amdgpu_buffer_rsrc_t ww = window(g.W + (size_t)n0 * K, ((size_t)(g.N - n0) * K) * 4);
    unsigned va[MB], vw[MB];
    int dst[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) {
        const int ra = min(r0 + 64 * i, M - 1 - m0);
        const int rw = min(r0 + 64 * i, g.N - 1 - n0);
        va[i] = ((unsigned)ra * K + kq * 4) * 4u;
        vw[i] = ((unsigned)rw * K + kq * 4) * 4u;
        dst[i] = (kq / 2) * HALF + swz(r0 + 64 * i, kq % 2);
    }
    const int nk = (K + BK - 1) / BK;
    float4 pal[MB], pau[MB], pw[MB];
    auto past = [&](int kt) { return !EXACT && kt * BK + kq * 4 >= K; };
    auto gload = [&](int kt) {
        const unsigned k = kt * (BK * 4u);
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            if (EXACT) {
                pal[i] = ld4(wal, va[i], k);
                pau[i] = ld4(wau, va[i], k);
                pw[i] = ld4(ww, vw[i], k);
            } else {
                const unsigned kk = past(kt) ? 0u : k;
                pal[i] = ld4(wal, va[i] + kk, 0);
                pau[i] = ld4(wau, va[i] + kk, 0);
                pw[i] = ld4(ww, vw[i] + kk, 0);
            }
        }
    };
    auto lstore = [&](int buf, int kt) {
        float *s = sm[buf];
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            if (past(kt)) pal[i] = pau[i] = pw[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4 *>(s + S_AL + dst[i]) = pal[i];
            *reinterpret_cast<float4 *>(s + S_AU + dst[i]) = pau[i];
            *reinterpret_cast<float4 *>(s + S_WP + dst[i]) = pos4(pw[i]);
            *reinterpret_cast<float4 *>(s + S_WN + dst[i]) = neg4(pw[i]);
        }
    };

    floatx16 cl[MB][MB], cu[MB][MB];
#pragma unroll
    for (int a = 0; a < MB; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;

    // fragments: lane (fi = lane % 32, fh = lane / 32) reads k = 8*ks + 4*fh .. +3 of row fi
    const int fi = lane % 32, fh = lane / 32;
    int fa[MB], fw[MB];
#pragma unroll
    for (int s = 0; s < MB; ++s) {
        fa[s] = swz((wm * MB + s) * 32 + fi, fh);
        fw[s] = swz((wn * MB + s) * 32 + fi, fh);
    }
    auto compute = [&](int buf, auto &&halfway) {
        const float *s = sm[buf];
#pragma unroll
        for (int ks = 0; ks < BK / 8; ++ks) {
            if (ks == 1) halfway();
            float4 al[MB], au[MB], wp[MB], wq[MB];
#pragma unroll
            for (int t = 0; t < MB; ++t) {
                al[t] = *reinterpret_cast<const float4 *>(s + S_AL + ks * HALF + fa[t]);
                au[t] = *reinterpret_cast<const float4 *>(s + S_AU + ks * HALF + fa[t]);
                wp[t] = *reinterpret_cast<const float4 *>(s + S_WP + ks * HALF + fw[t]);
                wq[t] = *reinterpret_cast<const float4 *>(s + S_WN + ks * HALF + fw[t]);
            }
#define FAITH_STEP(c)                                                           \
    _Pragma("unroll") for (int a = 0; a < MB; ++a) _Pragma("unroll") for (int b = 0; b < MB; ++b) { \
        cl[a][b] = mfma(al[a].c, wp[b].c, cl[a][b]);                            \
        cu[a][b] = mfma(au[a].c, wp[b].c, cu[a][b]);                            \
    }                                                                           \
    _Pragma("unroll") for (int a = 0; a < MB; ++a) _Pragma("unroll") for (int b = 0; b < MB; ++b) { \
        cl[a][b] = mfma(au[a].c, wq[b].c, cl[a][b]);                            \
        cu[a][b] = mfma(al[a].c, wq[b].c, cu[a][b]);                            \
    }
            FAITH_STEP(x)
            FAITH_STEP(y)
            FAITH_STEP(z)
            FAITH_STEP(w)
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

    // ---- epilogue: register r of a 32x32 block is row 8*(r/4) + 4*(lane/32) + r%4, column lane%32
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int col = n0 + (wn * MB + b) * 32 + fi;
        if (col >= g.N) continue;
#pragma unroll
        for (int a = 0; a < MB; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + (wm * MB + a) * 32 + 8 * (r / 4) + 4 * fh + (r % 4);
                if (row < M) {
                    const size_t o = (size_t)row * g.N + col;
                    __builtin_nontemporal_store(cl[a][b][r], &g.Cl[o]);
                    __builtin_nontemporal_store(cu[a][b][r], &g.Cu[o]);
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

__global__ void __launch_bounds__(256) signsplit_gemm_simple(const GemmArgs g) {
    __shared__ float sm[3 * 16 * 17];
    const int tiles_n = (g.N + 15) / 16;
    simple_tile(g, blockIdx.x / tiles_n, blockIdx.x % tiles_n, sm);
}

template <bool EXACT>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
signsplit_gemm(const GemmArgs g) {
    __shared__ float sm[2 * 4 * 2 * 128 * 8];            // two stages of four operands, 64 KB
    signsplit_gemm_body<EXACT, 2>(g, sm, blockIdx.x);
}
// Small problems: the first `b_tiles` workgroups take the 16 x 16 tiles of the constant-term rows
// (exact accumulation; each is a long chain of short steps, so they start first and run beside the
// MFMA tiles instead of in a launch of their own), the others a 64 x 64 MFMA tile each.
template <bool EXACT>
__global__ void __launch_bounds__(NTHREADS) signsplit_gemm_small(const GemmArgs g, const int b_tiles) {
    __shared__ float sm[2 * 4 * 2 * 64 * 8];             // 32 KB
    if ((int)blockIdx.x < b_tiles) {
        const int tiles_n = (g.N + 15) / 16;
        const int m_blk = blockIdx.x / tiles_n;
        if (m_blk < (g.Mb + 15) / 16) simple_tile(g, (g.Mw + 15) / 16 + m_blk, blockIdx.x % tiles_n, sm);
        return;
    }
    signsplit_gemm_body<EXACT, 1>(g, sm, blockIdx.x - b_tiles);
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
                      faith::aligned(W, 16) && 128LL * dim_out * 4 < 0xffffffffLL;   // 32-bit offsets in a tile
    if (fast) {
        // coefficient rows on MFMA, constant-term rows on the exact-accumulation kernel
        // 64 x 64 macro-tiles when 128 x 128 ones would leave compute units without work
        const long long big_tiles = ((mw + 127) / 128) * ((dim_y_out + 127) / 128);
        // (they run within 2 % of the large tiles even at configuration 2, so the switch point is not critical)
        const int tile = big_tiles < 2 * faith::compute_units() ? 64 : 128;
        const long long mblks = (mw + tile - 1) / tile;
        const long long grid = ((mblks + XCDS - 1) / XCDS) * XCDS * ((dim_y_out + tile - 1) / tile);
        FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        const bool exact = dim_out % BK == 0;
        const long long gridb = ((rows + 15) / 16) * ((dim_y_out + 15) / 16);
        if (tile == 64) {
            // constant-term tiles in front, rounded up to a multiple of 8 so that the MFMA tiles keep
            // their XCD (workgroup number mod 8)
            const long long b_tiles = (gridb + XCDS - 1) / XCDS * XCDS;
            FAITH_REQUIRE(grid + b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
            if (exact)
                hipLaunchKernelGGL(signsplit_gemm_small<true>, dim3((unsigned)(grid + b_tiles)), dim3(NTHREADS), 0, st, g,
                                   (int)b_tiles);
            else
                hipLaunchKernelGGL(signsplit_gemm_small<false>, dim3((unsigned)(grid + b_tiles)), dim3(NTHREADS), 0, st, g,
                                   (int)b_tiles);
        } else {
            if (exact)
                hipLaunchKernelGGL(signsplit_gemm<true>, dim3((unsigned)grid), dim3(NTHREADS), 0, st, g);
            else
                hipLaunchKernelGGL(signsplit_gemm<false>, dim3((unsigned)grid), dim3(NTHREADS), 0, st, g);
            GemmArgs gb = g;
            gb.Mw = 0;
            hipLaunchKernelGGL(signsplit_gemm_simple, dim3((unsigned)gridb), dim3(256), 0, st, gb);
        }
    } else {
        const long long grid = ((mw + 15) / 16 + (rows + 15) / 16) * ((dim_y_out + 15) / 16);
        FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_matmul_verification: grid too large");
        hipLaunchKernelGGL(signsplit_gemm_simple, dim3((unsigned)grid), dim3(256), 0, st, g);
    }
    return faith::check_launch("faith_matmul_verification");
}

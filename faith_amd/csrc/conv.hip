// Sign-split bound propagation through a 2-D convolution, as an implicit GEMM on fp32 MFMA.
//
// Semantics from the reference's verify_conv and its launcher
// (HandTunedKernels/convolution_verification.cu:124-138, :219-239): a positive tap multiplies the
// same-side bound, a non-positive tap the opposite one,
//     y_l = conv(x_l, W+) + conv(x_u, W-)        y_u = conv(x_u, W+) + conv(x_l, W-)
// applied to (lb, ub) with the real batch and to (lw, uw) with D_in as the batch.  NCHW,
// W [C_out, C_in, K, K], zero padding.  (The reference kernel itself is unfinished -- it drops
// the last K-tile, ignores the tile origin in its padding test and never stores; the arithmetic
// above is what it sets out to compute.)
//
// Computed in centre / radius form (W+ + W- = W, W+ - W- = |W|):
//     y_l = M - R,   y_u = M + R,   M = conv((x_l + x_u) / 2, W),   R = conv((x_u - x_l) / 2, |W|)
// -- two products per tap where the formula above has four.  Sum and difference of an input pair are formed
// once, by the thread that stages the patch (an out-of-image position is 0 in both), the halving is left to the
// epilogue (exact either way); |W| by the wavefront that reads the weight.
//
// Implicit GEMM:  C[co, p] = sum_k W[co, k] * X[k, p],  k = (ci, kh, kw),  p = output pixel.
// MFMA rows are output channels (W and |W|), MFMA columns are pixels (centre and radius of x), so lanes run along ow and every store is a contiguous run of a
// channel plane -- NCHW needs no transposition.
//
// Workgroup = 4 wavefronts on 128 channels x (4 output rows x 32 output columns) of one image;
// wavefront tile 64 channels x 2 rows.  The reduction walks C_in in chunks of 4 channels.  Per
// chunk the LDS holds
//   * the input patch, centres and radii: [2][4][(4-1)*stride + K][(32-1)*stride + K], out-of-image
//     positions stored as exact zeros (so padding contributes +0 to both products), each input
//     element fetched from global memory once and reused by up to K*K taps;
//   * the weight slab [128][4*K*K] (row padded to an odd length: conflict-free column reads).
// No im2col matrix is ever formed: the B fragment of tap (kh, kw) is the patch read at a
// shifted offset.  One MFMA K-pair is (ci, tap) on lanes 0-31 and (ci + 2, tap) on lanes 32-63,
// which turns the half-wave distinction into a per-lane constant offset.
//
// The constant-term path (batch images, 1/D_in of the work, O(1) cancelling terms) runs in a
// direct kernel that accumulates in double and adds the bias.
#include <type_traits>

#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TCO = 128;      // output channels per workgroup
constexpr int TR = 4;         // output rows per workgroup
constexpr int TC = 32;        // output columns per workgroup
constexpr int CC = 4;         // input channels per reduction chunk
constexpr int NTHREADS = 256;

struct ConvArgs {
    const float *xl, *xu;     // [N, Ci, H, W]
    const float *w;           // [Co, Ci, K, K]
    const float *bias;        // [Co] or nullptr
    float *yl, *yu;           // [N, Co, Ho, Wo]
    int N, Ci, H, W, Co, K, S, P, Ho, Wo;
    // 1: whole images dealt to the XCDs (image n to XCD n % 8).  Consecutive workgroups run on the eight XCDs in turn;
    // numbered along an image, its tiles land on different XCDs, each of which then writes every image's result in
    // pieces; this way an XCD reads an image (halo rows and all) through one L2 and writes its planes whole.
    int remap = 0;
};

__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
conv_signsplit(const ConvArgs g) {
    extern __shared__ float smem[];
    const int KK = g.K * g.K;
    const int prow = (TR - 1) * g.S + g.K, pcol = (TC - 1) * g.S + g.K;
    const int PP = prow * pcol;                  // one channel plane of the patch
    const int WS = (CC * KK) | 1;                // weight row length, odd
    float *sXl = smem;                           // [CC][prow][pcol]
    float *sXu = sXl + CC * PP;
    float *sW = sXu + CC * PP;                   // [TCO][WS]

    const int tcol = (g.Wo + TC - 1) / TC, trow = (g.Ho + TR - 1) / TR, tco = (g.Co + TCO - 1) / TCO;
    int pid = blockIdx.x;
    const int ow0 = (pid % tcol) * TC;  pid /= tcol;
    const int oh0 = (pid % trow) * TR;  pid /= trow;
    const int co0 = (pid % tco) * TCO;  pid /= tco;
    const int n = pid;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int wm = wv / 2, wn = wv % 2;          // wm: channel half, wn: row pair
    const int fi = lane % 32, fh = lane / 32;

    const int ih0 = oh0 * g.S - g.P, iw0 = ow0 * g.S - g.P;
    const size_t img = (size_t)g.H * g.W;
    const float *xl_n = g.xl + (size_t)n * g.Ci * img;
    const float *xu_n = g.xu + (size_t)n * g.Ci * img;

    // per-lane fragment offsets
    int xoff[2], woff[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) xoff[b] = fh * (CC / 2) * PP + ((wn * 2 + b) * g.S) * pcol + fi * g.S;
#pragma unroll
    for (int a = 0; a < 2; ++a) woff[a] = (wm * 64 + a * 32 + fi) * WS + fh * (CC / 2) * KK;

    floatx16 cl[2][2], cu[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;

    for (int c0 = 0; c0 < g.Ci; c0 += CC) {
        // ---- stage the patch: a wavefront per (channel, patch row), lanes along the row
        for (int rr = wv; rr < CC * prow; rr += NTHREADS / 64) {
            const int ci = c0 + rr / prow, pr = rr % prow;
            const int ih = ih0 + pr;
            const bool row_ok = ci < g.Ci && ih >= 0 && ih < g.H;
            const size_t rbase = (size_t)ci * img + (size_t)ih * g.W;
            for (int pc = lane; pc < pcol; pc += 64) {
                const int iw = iw0 + pc;
                const bool ok = row_ok && iw >= 0 && iw < g.W;
                const float vl = ok ? xl_n[rbase + iw] : 0.f, vu = ok ? xu_n[rbase + iw] : 0.f;
                sXl[rr * pcol + pc] = vl + vu;               // twice the centre
                sXu[rr * pcol + pc] = vu - vl;               // twice the radius
            }
        }
        // ---- stage the weight slab: CC*KK contiguous floats per output channel
        {
            const int per = CC * KK;
            for (int e = tid; e < TCO * per; e += NTHREADS) {
                const int co = e / per, kk = e % per;
                const bool ok = co0 + co < g.Co && c0 + kk / KK < g.Ci;
                sW[co * WS + kk] = ok ? g.w[((size_t)(co0 + co) * g.Ci + c0) * KK + kk] : 0.f;
            }
        }
        __syncthreads();

        // ---- multiply: (CC/2) channel pairs x K*K taps, 16 MFMAs each
        for (int cp = 0; cp < CC / 2; ++cp) {
            int tap = 0;
            for (int kh = 0; kh < g.K; ++kh) {
                for (int kw = 0; kw < g.K; ++kw, ++tap) {
                    const int xo = cp * PP + kh * pcol + kw;
                    const int wo = cp * KK + tap;
                    float wp[2], wq[2], xl[2], xu[2];        // w, |w|; centre and radius of x
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
                        wp[a] = sW[woff[a] + wo];
                        wq[a] = __builtin_fabsf(wp[a]);
                    }
#pragma unroll
                    for (int b = 0; b < 2; ++b) {
                        xl[b] = sXl[xoff[b] + xo];
                        xu[b] = sXu[xoff[b] + xo];
                    }
#pragma unroll
                    for (int a = 0; a < 2; ++a)
#pragma unroll
                        for (int b = 0; b < 2; ++b) {
                            cl[a][b] = mfma(wp[a], xl[b], cl[a][b]);
                            cu[a][b] = mfma(wq[a], xu[b], cu[a][b]);
                        }
                }
            }
        }
        __syncthreads();
    }

    // ---- epilogue: register r of a block is channel 8*(r/4) + 4*(lane/32) + r%4, pixel lane%32
    const int ow = ow0 + fi;
    if (ow >= g.Wo) return;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int oh = oh0 + wn * 2 + b;
        if (oh >= g.Ho) continue;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int co = co0 + wm * 64 + a * 32 + 8 * (r / 4) + 4 * fh + (r % 4);
                if (co < g.Co) {
                    const size_t o = (((size_t)n * g.Co + co) * g.Ho + oh) * g.Wo + ow;
                    __builtin_nontemporal_store(0.5f * (cl[a][b][r] - cu[a][b][r]), &g.yl[o]);      // centre - radius
                    __builtin_nontemporal_store(0.5f * (cl[a][b][r] + cu[a][b][r]), &g.yu[o]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------ 3x3, stride 1 fast path
// Same tiling with every extent a compile-time constant (patch 6 x 34, weight rows of 36 + 1),
// LDS double-buffered and a register prefetch across chunks: the global loads of chunk c+1 are
// issued before the MFMAs of chunk c, land in the other LDS buffer halfway through them, and ONE
// barrier per chunk (288 MFMAs per wavefront) publishes them.  Global addresses are buffer
// addresses: the per-thread offsets are fixed for the whole reduction, the chunk advances the
// wave-uniform base, and a patch element that lies in the padding carries an offset past the end of
// the buffer, which the hardware answers with zero -- no predicate, no select.
// Needs C_in % 4 == 0 and a 16-byte aligned weight pointer (float4 weight loads).
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t window(const void *base, size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0,
                                             (int)((bytes >> 32) ? 0xffffffffu : (unsigned)bytes), 0x00020000);
}
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
conv_signsplit_k3s1(const ConvArgs g) {
    constexpr int K = 3, KK = 9, PROW = TR - 1 + K, PCOL = TC - 1 + K, PP = PROW * PCOL;   // 6, 34, 204
    constexpr int WS = CC * KK + 1;                      // 37
    constexpr int NP = (CC * PP + NTHREADS - 1) / NTHREADS;          // patch elements per thread and bound: 4
    constexpr int NW4 = (TCO * CC * KK / 4 + NTHREADS - 1) / NTHREADS;   // weight float4 per thread: 5
    constexpr unsigned NOWHERE = 0xfffffff0u;            // a buffer offset the hardware answers with zero
    __shared__ float sXl[2][CC * PP];
    __shared__ float sXu[2][CC * PP];
    __shared__ float sW[2][TCO * WS];

    const int tcol = (g.Wo + TC - 1) / TC, trow = (g.Ho + TR - 1) / TR, tco = (g.Co + TCO - 1) / TCO;
    int pid = blockIdx.x;
    if (g.remap) {
        const int per = tcol * trow * tco, idx = pid / 8, x = pid % 8;
        pid = (idx / per * 8 + x) * per + idx % per;
    }
    const int ow0 = (pid % tcol) * TC;  pid /= tcol;
    const int oh0 = (pid % trow) * TR;  pid /= trow;
    const int co0 = (pid % tco) * TCO;  pid /= tco;
    const int n = pid;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int wm = wv / 2, wn = wv % 2;
    const int fi = lane % 32, fh = lane / 32;

    const int ih0 = oh0 - g.P, iw0 = ow0 - g.P;
    const int img = g.H * g.W;
    // one image of x (the entry point checks that it spans less than 4 GB) and the weight rows of this
    // channel block
    const size_t image = (size_t)g.Ci * img;
    const float *xl_n = g.xl + n * image, *xu_n = g.xu + n * image;
    const float *w_blk = g.w + (size_t)co0 * g.Ci * KK;
    const size_t w_bytes = (size_t)(g.Co - co0) * g.Ci * KK * 4;

    // ---- staging plan, fixed for the whole reduction: byte offsets inside a 4-channel slab
    unsigned poff[NP];
#pragma unroll
    for (int u = 0; u < NP; ++u) {
        const int e = tid + u * NTHREADS;
        const int ci = e / PP, r2 = e % PP, pr = r2 / PCOL, pc = r2 % PCOL;
        const int ih = ih0 + pr, iw = iw0 + pc;
        const bool ok = e < CC * PP && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
        poff[u] = ok ? (unsigned)(ci * img + ih * g.W + iw) * 4u : NOWHERE;
    }
    unsigned wsrc[NW4];
    int wdst[NW4];
#pragma unroll
    for (int u = 0; u < NW4; ++u) {
        const int e = tid + u * NTHREADS;
        const int co = e / 9, f = e % 9;
        const bool ok = e < TCO * 9;
        // rows past C_out re-read the last row; they are never stored
        wsrc[u] = ok ? (unsigned)(min(co, g.Co - 1 - co0) * g.Ci * KK + f * 4) * 4u : NOWHERE;
        wdst[u] = ok ? co * WS + f * 4 : -1;
    }
    float pxl[NP], pxu[NP];
    float4 pw[NW4];
    auto prefetch = [&](int c0) {
        const __amdgpu_buffer_rsrc_t rl = window(xl_n, image * 4), ru = window(xu_n, image * 4);
        const __amdgpu_buffer_rsrc_t rw = window(w_blk, w_bytes);
        const unsigned cx = (unsigned)c0 * img * 4u, cw = (unsigned)c0 * KK * 4u;
#pragma unroll
        for (int u = 0; u < NP; ++u) {
            pxl[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rl, poff[u], cx, 0));
            pxu[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ru, poff[u], cx, 0));
        }
#pragma unroll
        for (int u = 0; u < NW4; ++u) {
            const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(rw, wsrc[u], cw, 0);
            pw[u] = make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
        }
    };
    auto commit = [&](int buf) {
#pragma unroll
        for (int u = 0; u < NP; ++u) {
            const int e = tid + u * NTHREADS;
            if (e < CC * PP) {
                sXl[buf][e] = pxl[u] + pxu[u];               // twice the centre
                sXu[buf][e] = pxu[u] - pxl[u];               // twice the radius
            }
        }
#pragma unroll
        for (int u = 0; u < NW4; ++u) {
            if (wdst[u] >= 0) {
                sW[buf][wdst[u] + 0] = pw[u].x;
                sW[buf][wdst[u] + 1] = pw[u].y;
                sW[buf][wdst[u] + 2] = pw[u].z;
                sW[buf][wdst[u] + 3] = pw[u].w;
            }
        }
    };

    int xoff[2], woff[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) xoff[b] = fh * (CC / 2) * PP + (wn * 2 + b) * PCOL + fi;
#pragma unroll
    for (int a = 0; a < 2; ++a) woff[a] = (wm * 64 + a * 32 + fi) * WS + fh * (CC / 2) * KK;

    floatx16 cl[2][2], cu[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;

    // the MFMAs of one channel pair (cp) of the chunk in LDS buffer `buf`
    auto multiply = [&](int buf, int cp) {
#pragma unroll
        for (int tap = 0; tap < KK; ++tap) {
            const int xo = cp * PP + (tap / K) * PCOL + (tap % K);
            const int wo = cp * KK + tap;
            float wp[2], wq[2], xl[2], xu[2];                // w, |w|; centre and radius of x
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                wp[a] = sW[buf][woff[a] + wo];
                wq[a] = __builtin_fabsf(wp[a]);
            }
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                xl[b] = sXl[buf][xoff[b] + xo];
                xu[b] = sXu[buf][xoff[b] + xo];
            }
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    cl[a][b] = mfma(wp[a], xl[b], cl[a][b]);
                    cu[a][b] = mfma(wq[a], xu[b], cu[a][b]);
                }
        }
    };

    prefetch(0);
    commit(0);
    __syncthreads();
    int buf = 0;
    for (int c0 = 0; c0 + CC < g.Ci; c0 += CC) {
        prefetch(c0 + CC);
        __builtin_amdgcn_sched_barrier(0);         // the fetch goes first
        multiply(buf, 0);
        __builtin_amdgcn_sched_barrier(0);         // staging between the two halves of the MFMAs
        commit(buf ^ 1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(buf, 1);
        __syncthreads();
        buf ^= 1;
    }
    multiply(buf, 0);
    multiply(buf, 1);

    // ---- epilogue: register r of a block is channel 8*(r/4) + 4*(lane/32) + r%4, pixel lane%32.
    // Buffer stores into image n of the result (less than 2 GB with 128 channels to spare: the entry
    // point checks): the channel and the row of a register are a wave-uniform offset, the lane's own
    // offset (its pixel, its half of the channels) never changes, and channels past C_out fall outside
    // the window -- no address arithmetic and no predicate on the vector ALU.
    const int ow = ow0 + fi;
    if (ow >= g.Wo) return;
    const size_t plane = (size_t)g.Ho * g.Wo;
    const __amdgpu_buffer_rsrc_t wyl = window(g.yl + (size_t)n * g.Co * plane, (size_t)g.Co * plane * 4);
    const __amdgpu_buffer_rsrc_t wyu = window(g.yu + (size_t)n * g.Co * plane, (size_t)g.Co * plane * 4);
    const unsigned plane_b = (unsigned)plane * 4u;
    const unsigned vo = (unsigned)(4 * fh) * plane_b + (unsigned)ow * 4u;
    const int wvu = __builtin_amdgcn_readfirstlane(wv);        // the wavefront's number as a scalar
    const int wmu = wvu / 2, wnu = wvu % 2;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const int oh = oh0 + wnu * 2 + b;
        if (oh >= g.Ho) continue;
#pragma unroll
        for (int a = 0; a < 2; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned so = (unsigned)(co0 + wmu * 64 + a * 32 + 8 * (r / 4) + (r % 4)) * plane_b +
                                    (unsigned)(oh * g.Wo) * 4u;
                // y_l = centre - radius, y_u = centre + radius (the accumulators hold twice each)
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(0.5f * (cl[a][b][r] - cu[a][b][r])), wyl, vo, so, 2 /* non-temporal */);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(0.5f * (cl[a][b][r] + cu[a][b][r])), wyu, vo, so, 2);
            }
        }
    }
}

// ------------------------------------------------------------------ other common layers, same scheme
// The straight-line, double-buffered kernel above with its extents as template parameters: kernel size K,
// stride S, input channels per reduction chunk CCH (a 1 x 1 layer has one tap per channel, so it takes 16
// channels a chunk to give a barrier 128 MFMAs; 3 x 3 and 5 x 5 take 4), and whether a row of the weight
// slab can be fetched 16 bytes at a time (WVEC: C_in % 4 == 0, aligned) or needs 4-byte loads (the first
// layer of an image classifier has C_in = 3).  Channels past C_in need no predicate on either operand: the
// input window ends with the image's last channel, so such a patch element reads as zero, and a zero patch
// makes whatever finite weight the slab holds at that position irrelevant.
//
// The tile is a parameter too.  An MFMA block is 32 channels x 32 pixels; the 32 pixels are TCB columns x 32 / TCB
// rows of the image (TCB = 32: one row; 16: two rows of a 16-wide image, which a 32-column tile would fill by
// half), and the workgroup's four wavefronts are WM x 4 / WM over (halves of 64 channels) x (pairs of pixel
// blocks): WM = 2 is 128 channels x 4 blocks, WM = 1 is 64 channels x 8 blocks for layers of up to 64 channels.
// A wavefront holds MA x MB blocks (channels x pixels).  2 x 2 -- 128 accumulator registers, two wavefronts per
// SIMD -- has the most reuse of what is read from LDS and suits long reductions.  A layer with a short reduction
// is mostly the stream of its results; its workgroups fetch, multiply and store in phases, and with only two of them
// on a CU the phases of the whole machine fall together (the MFMA pipe idles while everything stores).  1 x 2
// blocks (64 accumulators) let four workgroups share a CU, whose phases then overlap.
template <int K, int S, int CCH, bool WVEC, int TCB, int WM, int MA = 2, int MB = 2>
struct FastTile {
    static constexpr int RPB = 32 / TCB;                 // image rows of one pixel block
    static constexpr int NPB = MB * (4 / WM);            // pixel blocks of a workgroup
    static constexpr int ROWS = NPB * RPB, CHANNELS = 32 * MA * WM;
    // wavefronts per SIMD the register budget is set for: two with 128 accumulators, four with 64 -- three where the
    // patch of a strided or 5 x 5 layer needs more than 128 registers beside them
    static constexpr int WAVES = MA * MB == 4 ? 2 : (S > 1 || K >= 5) ? 3 : 4;
    static constexpr int KK = K * K, PROW = (ROWS - 1) * S + K, PCOL = (TCB - 1) * S + K, PP = PROW * PCOL;
    static constexpr int WS = (CCH * KK) | 1;
    static constexpr size_t LDS = ((size_t)4 * CCH * PP + (size_t)2 * CHANNELS * WS) * sizeof(float);
};

template <int K, int S, int CCH, bool WVEC, int TCB, int WM, int MA = 2, int MB = 2>
__global__ void __launch_bounds__(NTHREADS)
    __attribute__((amdgpu_waves_per_eu(FastTile<K, S, CCH, WVEC, TCB, WM, MA, MB>::WAVES, FastTile<K, S, CCH, WVEC, TCB, WM, MA, MB>::WAVES)))
conv_signsplit_fast(const ConvArgs g, const int total_tiles) {
    using T = FastTile<K, S, CCH, WVEC, TCB, WM, MA, MB>;
    constexpr int TCO = T::CHANNELS, TR = T::ROWS, TC = TCB, RPB = T::RPB;      // shadow the file-scope tile
    constexpr int KK = K * K, PROW = T::PROW, PCOL = T::PCOL, PP = T::PP;
    constexpr int WROW = CCH * KK;                       // floats of one weight row in a chunk
    constexpr int WS = WROW | 1;                         // padded to an odd length: conflict-free column reads
    constexpr int NP = (CCH * PP + NTHREADS - 1) / NTHREADS;             // patch elements per thread and bound
    constexpr int WPT = WVEC ? 4 : 1;                                    // floats per weight load
    constexpr int NWL = (TCO * WROW / WPT + NTHREADS - 1) / NTHREADS;    // weight loads per thread
    constexpr unsigned NOWHERE = 0xfffffff0u;            // a buffer offset the hardware answers with zero
    static_assert(CCH % 4 == 0 && WROW % 4 == 0, "a chunk is split into two halves of channel pairs");
    extern __shared__ float smem[];
    float *sXl = smem;                                   // [2][CCH * PP]
    float *sXu = sXl + 2 * CCH * PP;
    float *sW = sXu + 2 * CCH * PP;                      // [2][TCO * WS]

    const int tcol = (g.Wo + TC - 1) / TC, trow = (g.Ho + TR - 1) / TR, tco = (g.Co + TCO - 1) / TCO;
    // Persistent: the grid is sized to the machine and a workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x,
    // ...  The layers this kernel serves have short reductions (a 1 x 1 layer: four chunks), so a tile is mostly
    // its first fetch and its 128 KB of results; in a walk the stores of one tile drain while the next is fetched
    // and multiplied, where one-tile workgroups load, multiply and store in step with each other (1 x 1 64 -> 128:
    // 113 -> 107 us, 3 x 3 3 -> 64: 54.4 -> 51.7 us; the longer reductions are unchanged).  Fetching the next tile's
    // first chunk before the last MFMAs of the current one as well measured no better (105 / 53.8 us).
    for (int tile = blockIdx.x; tile < total_tiles; tile += gridDim.x) {
    int pid = tile;
    if (g.remap) {
        const int per = tcol * trow * tco, idx = pid / 8, x = pid % 8;
        pid = (idx / per * 8 + x) * per + idx % per;
    }
    const int ow0 = (pid % tcol) * TC;  pid /= tcol;
    const int oh0 = (pid % trow) * TR;  pid /= trow;
    const int co0 = (pid % tco) * TCO;  pid /= tco;
    const int n = pid;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int wm = wv / (4 / WM), wn = wv % (4 / WM);
    const int fi = lane % 32, fh = lane / 32;
    const int fr = fi / TCB, fc = fi % TCB;              // the lane's pixel inside a block: row, column

    const int ih0 = oh0 * S - g.P, iw0 = ow0 * S - g.P;
    const int img = g.H * g.W;
    const size_t image = (size_t)g.Ci * img;
    const float *xl_n = g.xl + n * image, *xu_n = g.xu + n * image;
    const float *w_blk = g.w + (size_t)co0 * g.Ci * KK;
    const size_t w_bytes = (size_t)(g.Co - co0) * g.Ci * KK * 4;

    // ---- staging plan, fixed for the whole reduction: byte offsets inside a chunk of channels
    // (kept in registers by the 1 x 1 layers and by the 3 x 3 layers with 128 accumulators and at most 12 patch
    // elements per thread -- stride 2, 64 -> 128: 183 us with the plan, 197 us without; 4 x 4 and 5 x 5 layers have
    // no registers to spare for it beside their weight slab, nor have the stride-2 tiles of 64 channels, whose patch
    // is 18 elements per thread, nor tiles with a smaller register budget: they work each offset out again where it
    // is used, a dozen integer operations per element against hundreds of MFMAs per chunk)
    constexpr bool KEEP_PLAN = K < 4 && NP <= 12 && (T::WAVES == 2 || K == 1);
    auto patch_offset = [&](int u, int tid_) -> unsigned {
        const int e = tid_ + u * NTHREADS;
        const int ci = e / PP, r2 = e % PP, pr = r2 / PCOL, pc = r2 % PCOL;
        const int ih = ih0 + pr, iw = iw0 + pc;
        const bool ok = e < CCH * PP && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
        return ok ? (unsigned)(ci * img + ih * g.W + iw) * 4u : NOWHERE;
    };
    unsigned poff[KEEP_PLAN ? NP : 1];
    if constexpr (KEEP_PLAN) {
#pragma unroll
        for (int u = 0; u < NP; ++u) poff[u] = patch_offset(u, tid);
    }
    // weight load u of a thread: element e = tid + u * NTHREADS of the slab, row e / (WROW / WPT); its source and
    // destination are a few integer operations on compile-time divisors, recomputed where they are used so
    // that they do not occupy 2 NWL registers across the MFMAs (rows past C_out re-read the last row; they are
    // never stored)
    const int last_row = g.Co - 1 - co0;
    // (the empty asm makes the thread number opaque inside a chunk: otherwise the compiler hoists all 2 NWL values
    // out of the reduction loop again)
    auto wsrc = [&](int u, int tid_) -> unsigned {
        const int e = tid_ + u * NTHREADS;
        const int co = e / (WROW / WPT), f = e % (WROW / WPT);
        return e < TCO * (WROW / WPT) ? (unsigned)(min(co, last_row) * g.Ci * KK + f * WPT) * 4u : NOWHERE;
    };
    auto wdst = [&](int u, int tid_) -> int {
        const int e = tid_ + u * NTHREADS;
        return e < TCO * (WROW / WPT) ? (e / (WROW / WPT)) * WS + (e % (WROW / WPT)) * WPT : -1;
    };
    // A large weight slab (5 x 5: 50 floats per thread and chunk) is fetched in two parts so that its registers
    // fit beside the 128 accumulators: part 1 with the patch, before the first half of the MFMAs, part 2 after
    // the first part has gone to LDS, before the second half.
    constexpr bool TWO_PARTS = NWL * WPT > 32;
    constexpr int NW1 = TWO_PARTS ? (NWL + 1) / 2 : NWL, NW2 = NWL - NW1, NWR = NW1 > NW2 ? NW1 : NW2;
    float pxl[NP], pxu[NP];
    float pw[NWR][WPT];
    auto fetch_patch = [&](int c0) {
        const __amdgpu_buffer_rsrc_t rl = window(xl_n, image * 4), ru = window(xu_n, image * 4);
        const unsigned cx = (unsigned)c0 * img * 4u;
        int tid_ = tid;
        if constexpr (!KEEP_PLAN) asm volatile("" : "+v"(tid_));     // opaque: the offsets are not hoisted out of the loop
#pragma unroll
        for (int u = 0; u < NP; ++u) {
            const unsigned off = KEEP_PLAN ? poff[KEEP_PLAN ? u : 0] : patch_offset(u, tid_);
            pxl[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rl, off, cx, 0));
            pxu[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(ru, off, cx, 0));
        }
    };
    auto fetch_weights = [&](int c0, auto first, auto count) {
        const __amdgpu_buffer_rsrc_t rw = window(w_blk, w_bytes);
        const unsigned cw = (unsigned)c0 * KK * 4u;
        int tid_ = tid;
        asm volatile("" : "+v"(tid_));
#pragma unroll
        for (int u = 0; u < decltype(count)::value; ++u) {
            if constexpr (WVEC) {
                const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(rw, wsrc(u + decltype(first)::value, tid_), cw, 0);
                pw[u][0] = __uint_as_float(v.x);
                pw[u][1] = __uint_as_float(v.y);
                pw[u][2] = __uint_as_float(v.z);
                pw[u][3] = __uint_as_float(v.w);
            } else {
                pw[u][0] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rw, wsrc(u + decltype(first)::value, tid_), cw, 0));
            }
        }
    };
    auto commit_patch = [&](int buf) {
        float *dl = sXl + buf * CCH * PP, *du = sXu + buf * CCH * PP;
#pragma unroll
        for (int u = 0; u < NP; ++u) {
            const int e = tid + u * NTHREADS;
            if (e < CCH * PP) {
                dl[e] = pxl[u] + pxu[u];                     // twice the centre
                du[e] = pxu[u] - pxl[u];                     // twice the radius
            }
        }
    };
    auto commit_weights = [&](int buf, auto first, auto count) {
        float *dw = sW + buf * TCO * WS;
        int tid_ = tid;
        asm volatile("" : "+v"(tid_));
#pragma unroll
        for (int u = 0; u < decltype(count)::value; ++u) {
            const int d = wdst(u + decltype(first)::value, tid_);
            if (d >= 0) {
#pragma unroll
                for (int q = 0; q < WPT; ++q) dw[d + q] = pw[u][q];
            }
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, NW1>;
    using I2 = std::integral_constant<int, NW2>;

    int xoff[MB], woff[MA];
#pragma unroll
    for (int b = 0; b < MB; ++b) xoff[b] = fh * (CCH / 2) * PP + (((wn * MB + b) * RPB + fr) * S) * PCOL + fc * S;
#pragma unroll
    for (int a = 0; a < MA; ++a) woff[a] = ((wm * MA + a) * 32 + fi) * WS + fh * (CCH / 2) * KK;

    floatx16 cl[MA][MB], cu[MA][MB];
#pragma unroll
    for (int a = 0; a < MA; ++a)
#pragma unroll
        for (int b = 0; b < MB; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][b][r] = cu[a][b][r] = 0.f;

    // the MFMAs of channel pairs [cp0, cp1) of the chunk in LDS buffer `buf`
    auto multiply = [&](int buf, int cp0, int cp1) {
        const float *bl = sXl + buf * CCH * PP, *bu = sXu + buf * CCH * PP, *bw = sW + buf * TCO * WS;
#pragma unroll
        for (int cp = cp0; cp < cp1; ++cp) {
#pragma unroll
            for (int tap = 0; tap < KK; ++tap) {
                const int xo = cp * PP + (tap / K) * PCOL + (tap % K);
                const int wo = cp * KK + tap;
                float wp[MA], wq[MA], xl[MB], xu[MB];        // w, |w|; centre and radius of x
#pragma unroll
                for (int a = 0; a < MA; ++a) {
                    wp[a] = bw[woff[a] + wo];
                    wq[a] = __builtin_fabsf(wp[a]);
                }
#pragma unroll
                for (int b = 0; b < MB; ++b) {
                    xl[b] = bl[xoff[b] + xo];
                    xu[b] = bu[xoff[b] + xo];
                }
#pragma unroll
                for (int a = 0; a < MA; ++a)
#pragma unroll
                    for (int b = 0; b < MB; ++b) {
                        cl[a][b] = mfma(wp[a], xl[b], cl[a][b]);
                        cu[a][b] = mfma(wq[a], xu[b], cu[a][b]);
                    }
            }
        }
    };

    fetch_patch(0);
    fetch_weights(0, I0{}, I1{});
    commit_patch(0);
    commit_weights(0, I0{}, I1{});
    if constexpr (TWO_PARTS) {
        fetch_weights(0, I1{}, I2{});
        commit_weights(0, I1{}, I2{});
    }
    __syncthreads();
    int buf = 0;
    for (int c0 = 0; c0 + CCH < g.Ci; c0 += CCH) {
        fetch_patch(c0 + CCH);
        fetch_weights(c0 + CCH, I0{}, I1{});
        __builtin_amdgcn_sched_barrier(0);         // the fetch goes first
        multiply(buf, 0, CCH / 4);
        __builtin_amdgcn_sched_barrier(0);         // staging between the two halves of the MFMAs
        commit_patch(buf ^ 1);
        commit_weights(buf ^ 1, I0{}, I1{});
        if constexpr (TWO_PARTS) fetch_weights(c0 + CCH, I1{}, I2{});
        __builtin_amdgcn_sched_barrier(0);
        multiply(buf, CCH / 4, CCH / 2);
        if constexpr (TWO_PARTS) {
            __builtin_amdgcn_sched_barrier(0);
            commit_weights(buf ^ 1, I1{}, I2{});
        }
        __syncthreads();
        buf ^= 1;
    }
    multiply(buf, 0, CCH / 2);

    // ---- epilogue: as in the 3 x 3 stride-1 kernel (buffer stores into image n of the result); a lane whose
    // pixel lies outside the image carries an offset outside the window
    const size_t plane = (size_t)g.Ho * g.Wo;
    const __amdgpu_buffer_rsrc_t wyl = window(g.yl + (size_t)n * g.Co * plane, (size_t)g.Co * plane * 4);
    const __amdgpu_buffer_rsrc_t wyu = window(g.yu + (size_t)n * g.Co * plane, (size_t)g.Co * plane * 4);
    const unsigned plane_b = (unsigned)plane * 4u;
    const int wvu = __builtin_amdgcn_readfirstlane(wv);
    const int wmu = wvu / (4 / WM), wnu = wvu % (4 / WM);
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int row0 = oh0 + (wnu * MB + b) * RPB;                 // first image row of this pixel block
        if (row0 >= g.Ho) continue;
        const bool inside = ow0 + fc < g.Wo && row0 + fr < g.Ho;
        const unsigned vo = inside ? (unsigned)(4 * fh) * plane_b + (unsigned)(fr * g.Wo + ow0 + fc) * 4u : 0x80000000u;
#pragma unroll
        for (int a = 0; a < MA; ++a) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned so = (unsigned)(co0 + (wmu * MA + a) * 32 + 8 * (r / 4) + (r % 4)) * plane_b +
                                    (unsigned)(row0 * g.Wo) * 4u;
                // y_l = centre - radius, y_u = centre + radius (the accumulators hold twice each)
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(0.5f * (cl[a][b][r] - cu[a][b][r])), wyl, vo, so, 2 /* non-temporal */);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(0.5f * (cl[a][b][r] + cu[a][b][r])), wyu, vo, so, 2);
            }
        }
    }
    __syncthreads();                               // the next tile's first chunk goes into the buffers just read
    }
}

template <int K, int S, int CCH, bool WVEC, int TCB, int WM, int MA = 2, int MB = 2>
bool launch_tile(const ConvArgs &g, hipStream_t st) {
    using T = FastTile<K, S, CCH, WVEC, TCB, WM, MA, MB>;
    static_assert(T::LDS <= 160 * 1024, "the two LDS stages of this instantiation do not fit a workgroup");
    const long long grid = (long long)g.N * ((g.Co + T::CHANNELS - 1) / T::CHANNELS) * ((g.Ho + T::ROWS - 1) / T::ROWS) *
                           ((g.Wo + TCB - 1) / TCB);
    if (grid > 0x7fffffffLL) return false;
    if (!faith::reserve_lds(conv_signsplit_fast<K, S, CCH, WVEC, TCB, WM, MA, MB>, T::LDS)) return false;
    // workgroups a CU holds: one wavefront of each on every SIMD (registers), and their LDS
    const long long by_lds = (160 * 1024) / (long long)T::LDS;
    const long long resident = (by_lds < T::WAVES ? by_lds : T::WAVES) * faith::compute_units();
    const long long launched = grid < resident ? grid : resident;
    ConvArgs h = g;
    h.remap = (g.N % 8 == 0 && launched % 8 == 0 && faith::tune_get(FAITH_TUNE_CONV_VARIANT) != 2) ? 1 : 0;
    hipLaunchKernelGGL((conv_signsplit_fast<K, S, CCH, WVEC, TCB, WM, MA, MB>), dim3((unsigned)launched), dim3(NTHREADS), T::LDS,
                       st, h, (int)grid);
    return true;
}

// Tile for this layer: 16-column pixel blocks when the last (or only) 32-column tile of a row would be at most
// half full, 64-channel workgroups when the last (or only) 128-channel tile would be.
template <int K, int S, int CCH, bool WVEC>
bool launch_fast(const ConvArgs &g, hipStream_t st) {
    const bool narrow = (g.Wo - 1) % 32 < 16, few = (g.Co - 1) % 128 < 64;
    // at most 32 output channels: 32 channels x 8 pixel blocks, one channel block per wavefront (a 64-channel tile
    // would multiply zeros for half of its rows: 3 x 3 16 -> 32 92 -> 52 us, 32 -> 32 171 -> 104 us, 5 x 5 16 -> 32
    // 227 -> 126 us on 256 images of 32 x 32; with 1 x 4 blocks per wavefront instead of 1 x 2: no better).  Layers
    // of 65 ... 96 channels keep the 64-channel tiles: three 32-channel tiles read the patch three times and measured
    // slower (3 x 3 stride 2 32 -> 96: 121 against 98 us).
    if (g.Co <= 32) return narrow ? launch_tile<K, S, CCH, WVEC, 16, 1, 1, 2>(g, st) : launch_tile<K, S, CCH, WVEC, 32, 1, 1, 2>(g, st);
    // results of at most 8 x 8 pixels (the last layers of a small classifier): pixel blocks of 8 columns x 4 rows, two
    // of them a tile -- the whole image --, under 128 or 64 channels (against 16-column blocks, which such an image
    // fills by half: 3 x 3 64 -> 128 110 -> 76 us, 128 -> 128 208 -> 145 us, 4 x 4 stride 2 32 -> 64 102 -> 50 us)
    if (g.Wo <= 8 && g.Ho <= 8)
        return g.Co > 64 ? launch_tile<K, S, CCH, WVEC, 8, 4, 1, 2>(g, st) : launch_tile<K, S, CCH, WVEC, 8, 2, 1, 1>(g, st);
    if (narrow && few) return launch_tile<K, S, CCH, WVEC, 16, 1>(g, st);
    if (narrow) return launch_tile<K, S, CCH, WVEC, 16, 2>(g, st);
    if (few) return launch_tile<K, S, CCH, WVEC, 32, 1>(g, st);
    return launch_tile<K, S, CCH, WVEC, 32, 2>(g, st);
}

// Layers whose reduction is short (at most 64 products per result: a 1 x 1 layer of up to 64 channels, the 3 x 3
// first layer of an image classifier): 1 x 2 blocks per wavefront, four workgroups per CU (see FastTile) --
// 64 channels x 4 pixel blocks, 128 channels x 2 pixel blocks where the layer has that many channels (the
// patch is then read once instead of twice), or 32 channels x 8 pixel blocks (below).  Measured against 2 x 2 blocks: 1 x 1 64 -> 128 107 -> 96-99 us,
// 1 x 1 32 -> 64 49 -> 41 us, 3 x 3 3 -> 64 45 -> 39-41 us; one block per wavefront was no faster than two.
template <int K, int S, int CCH, bool WVEC>
bool launch_brief(const ConvArgs &g, hipStream_t st) {
    if ((g.Wo - 1) % 32 < 16) return launch_tile<K, S, CCH, WVEC, 16, 2, 1, 2>(g, st);
    // 3 x 3 first layers whose last (or only) 64 channels would be at most half there: 32 channels x 8 pixel
    // blocks, the four wavefronts side by side over the image rows (3 -> 32: 35 -> 23 us, 3 -> 96: 73 -> 53 us,
    // 3 -> 64 the same either way).  Not for 1 x 1 layers, whose patch of 8 rows x 16 channels a chunk would leave
    // room for two workgroups on a CU instead of four (1 x 1 64 -> 128 on it: 165 against 96 us).
    if constexpr (K == 3) {
        if ((g.Co - 1) % 64 < 32) return launch_tile<K, S, CCH, WVEC, 32, 1, 1, 2>(g, st);
    }
    if ((g.Co - 1) % 128 >= 64) return launch_tile<K, S, CCH, WVEC, 32, 4, 1, 2>(g, st);
    return launch_tile<K, S, CCH, WVEC, 32, 2, 1, 2>(g, st);
}

// The straight-line instantiation for this layer, if there is one: 3 x 3 at stride 1 or 2, 1 x 1, 5 x 5.
bool dispatch_fast(const ConvArgs &g, bool wvec, hipStream_t st) {
    const int key = g.K * 10 + g.S;
    const bool brief = g.Ci * g.K * g.K <= 64 && faith::tune_get(FAITH_TUNE_CONV_VARIANT) != 3;
    if (brief) {
        if (key == 11) return wvec ? launch_brief<1, 1, 16, true>(g, st) : launch_brief<1, 1, 16, false>(g, st);
        if (key == 31 && !wvec) return launch_brief<3, 1, 4, false>(g, st);
    }
    if (wvec) {
        switch (key) {
            case 31: return launch_fast<3, 1, 4, true>(g, st);      // layers that fill 128 x (4 x 32) tiles take the kernel above
            case 32: return launch_fast<3, 2, 4, true>(g, st);
            case 11: return launch_fast<1, 1, 16, true>(g, st);
            case 51: return launch_fast<5, 1, 4, true>(g, st);
            case 42: return launch_fast<4, 2, 4, true>(g, st);      // the 4 x 4 stride-2 layers of the small image classifiers
            case 41: return launch_fast<4, 1, 4, true>(g, st);
            default: return false;
        }
    }
    switch (key) {
        case 31: return launch_fast<3, 1, 4, false>(g, st);
        case 32: return launch_fast<3, 2, 4, false>(g, st);
        case 11: return launch_fast<1, 1, 16, false>(g, st);
        case 51: return launch_fast<5, 1, 4, false>(g, st);
        case 42: return launch_fast<4, 2, 4, false>(g, st);
        case 41: return launch_fast<4, 1, 4, false>(g, st);
        default: return false;
    }
}

// Direct convolution for the constant terms: 32 neighbouring outputs x 4 output channels x 8 groups of
// input channels per workgroup; a thread sums its share of the input channels in double (an fp32 x fp32
// product is exact there) for its pixel and four output channels -- the centre and the radius of an input
// value are formed once and serve all four --, the 8 partial sums meet in LDS, one rounding, then the bias.
constexpr int DP = 32, DG = 8, DC = 4;
__global__ void __launch_bounds__(DP * DG) conv_direct(const ConvArgs g) {
    __shared__ double red[2][DC][DG][DP];
    const int cob = (g.Co + DC - 1) / DC;                     // blocks of output channels
    const size_t total = (size_t)g.N * cob * g.Ho * g.Wo;
    const int px = threadIdx.x % DP, cg = threadIdx.x / DP;
    const size_t idx = (size_t)blockIdx.x * DP + px;
    const bool live = idx < total;
    const size_t id = live ? idx : total - 1;
    const int ow = id % g.Wo;
    const int oh = (id / g.Wo) % g.Ho;
    const int co0 = (int)((id / ((size_t)g.Wo * g.Ho)) % cob) * DC;
    const int n = id / ((size_t)g.Wo * g.Ho * cob);
    const int KK = g.K * g.K;
    double sm[DC], sr[DC];
#pragma unroll
    for (int c = 0; c < DC; ++c) sm[c] = sr[c] = 0.0;
    for (int ci = cg; ci < g.Ci; ci += DG) {
        const float *xl = g.xl + ((size_t)n * g.Ci + ci) * g.H * g.W;
        const float *xu = g.xu + ((size_t)n * g.Ci + ci) * g.H * g.W;
        const float *w = g.w + ((size_t)co0 * g.Ci + ci) * KK;
        const size_t w_step = (size_t)g.Ci * KK;              // one output channel further
        for (int kh = 0; kh < g.K; ++kh) {
            const int ih = oh * g.S - g.P + kh;
            if (ih < 0 || ih >= g.H) continue;
            for (int kw = 0; kw < g.K; ++kw) {
                const int iw = ow * g.S - g.P + kw;
                if (iw < 0 || iw >= g.W) continue;
                // w+ a + w- b = w m - |w| r and w+ b + w- a = w m + |w| r with m = (a + b) / 2,
                // r = (b - a) / 2, both exact in double: two fused multiply-adds per tap instead of four
                const double a = xl[ih * g.W + iw], b = xu[ih * g.W + iw];
                const double m = 0.5 * (a + b), r = 0.5 * (b - a);
#pragma unroll
                for (int c = 0; c < DC; ++c) {
                    // channels past C_out re-read the last one; their sums are never stored
                    const double wv = w[(size_t)min(c, g.Co - 1 - co0) * w_step + kh * g.K + kw];
                    sm[c] += wv * m;
                    sr[c] += fabs(wv) * r;
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < DC; ++c) {
        red[0][c][cg][px] = sm[c] - sr[c];
        red[1][c][cg][px] = sm[c] + sr[c];
    }
    __syncthreads();
    // thread (cg, px) finishes output channel co0 + cg of its pixel (cg < DC)
    if (cg < DC && live && co0 + cg < g.Co) {
        double sl = red[0][cg][0][px], su = red[1][cg][0][px];
#pragma unroll
        for (int c = 1; c < DG; ++c) {
            sl += red[0][cg][c][px];
            su += red[1][cg][c][px];
        }
        const int co = co0 + cg;
        const float add = g.bias ? g.bias[co] : 0.f;
        const size_t o = (((size_t)n * g.Co + co) * g.Ho + oh) * g.Wo + ow;
        g.yl[o] = (float)sl + add;
        g.yu[o] = (float)su + add;
    }
}

}  // namespace

extern "C" int faith_convolution_verification(const float *x_lb, const float *x_ub, const float *x_lw,
                                              const float *x_uw, const float *W, const float *bias, float *y_lb,
                                              float *y_ub, float *y_lw, float *y_uw, int batch_size, int Height,
                                              int Width, int CIN, int COUT, int K, int Stride, int padding_size,
                                              int dim_in, void *stream) {
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(W);
    FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(W);
    FAITH_ALIGNED4(bias); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_REQUIRE(batch_size > 0 && Height > 0 && Width > 0 && CIN > 0 && COUT > 0 && K > 0 && Stride > 0 &&
                      padding_size >= 0 && dim_in > 0,
                  FAITH_ERR_SHAPE,
                  "faith_convolution_verification: batch=%d H=%d W=%d CIN=%d COUT=%d K=%d stride=%d pad=%d dim_in=%d",
                  batch_size, Height, Width, CIN, COUT, K, Stride, padding_size, dim_in);
    const int Ho = (Height + 2 * padding_size - K) / Stride + 1, Wo = (Width + 2 * padding_size - K) / Stride + 1;
    FAITH_REQUIRE(Height + 2 * padding_size >= K && Width + 2 * padding_size >= K && Ho > 0 && Wo > 0,
                  FAITH_ERR_SHAPE, "faith_convolution_verification: kernel %d larger than the padded input", K);
    hipStream_t st = static_cast<hipStream_t>(stream);

    // coefficients: D_in images through the MFMA kernel
    ConvArgs gw{x_lw, x_uw, W, nullptr, y_lw, y_uw, dim_in, CIN, Height, Width, COUT, K, Stride, padding_size, Ho, Wo};
    const int prow = (TR - 1) * Stride + K, pcol = (TC - 1) * Stride + K;
    const size_t smem = ((size_t)2 * CC * prow * pcol + (size_t)TCO * ((CC * K * K) | 1)) * sizeof(float);
    FAITH_REQUIRE(smem <= 160 * 1024, FAITH_ERR_UNSUPPORTED,
                  "faith_convolution_verification: K=%d stride=%d needs %zu bytes of LDS per workgroup (limit 163840)",
                  K, Stride, smem);
    if (smem > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(conv_signsplit),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        FAITH_REQUIRE(e == hipSuccess, FAITH_ERR_LAUNCH, "faith_convolution_verification: cannot reserve %zu bytes of LDS (%s)",
                      smem, hipGetErrorString(e));
    }
    const long long grid = (long long)dim_in * ((COUT + TCO - 1) / TCO) * ((Ho + TR - 1) / TR) * ((Wo + TC - 1) / TC);
    FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_convolution_verification: grid too large");
    const bool k3s1 = K == 3 && Stride == 1 && CIN % 4 == 0 && faith::aligned(W, 16) &&
                      (long long)CIN * Height * Width * 4 < 0xfffffff0LL &&      // 32-bit byte offsets inside an image
                      (long long)128 * CIN * 9 * 4 + (long long)CIN * 9 * 4 < 0xfffffff0LL &&  // and inside a block of weight rows
                      ((long long)COUT + 132) * Ho * Wo * 4 < 0x80000000LL;                   // and inside an image of the result
    // the limits of 32-bit byte offsets, for any kernel size: inside an image of x, inside a block of 128 weight
    // rows plus one chunk, inside an image of the result
    const bool offsets_fit = (long long)CIN * Height * Width * 4 < 0xfffffff0LL &&
                             (long long)129 * CIN * K * K * 4 + 64LL * K * K * 4 < 0xfffffff0LL &&
                             ((long long)COUT + 132) * Ho * Wo * 4 < 0x80000000LL;
    const bool wvec = CIN % 4 == 0 && faith::aligned(W, 16);
    const int forced = faith::tune_get(FAITH_TUNE_CONV_VARIANT);      // 1: the general kernel, whatever the layer
    const bool full_tiles = (Wo - 1) % 32 >= 16 && (COUT - 1) % 128 >= 64;     // else a smaller tile wastes less
    if (k3s1 && full_tiles && forced != 1) {
        gw.remap = (dim_in % 8 == 0 && forced != 2) ? 1 : 0;
        hipLaunchKernelGGL(conv_signsplit_k3s1, dim3((unsigned)grid), dim3(NTHREADS), 0, st, gw);
        gw.remap = 0;
    }
    else if (!(forced != 1 && offsets_fit && dispatch_fast(gw, wvec, st)))
        hipLaunchKernelGGL(conv_signsplit, dim3((unsigned)grid), dim3(NTHREADS), smem, st, gw);

    // constant terms: batch images through the exact-accumulation kernel, bias added
    ConvArgs gb{x_lb, x_ub, W, bias, y_lb, y_ub, batch_size, CIN, Height, Width, COUT, K, Stride, padding_size, Ho, Wo};
    const long long nb = (long long)batch_size * ((COUT + DC - 1) / DC) * Ho * Wo;
    hipLaunchKernelGGL(conv_direct, dim3((unsigned)((nb + DP - 1) / DP)), dim3(DP * DG), 0, st, gb);
    return faith::check_launch("faith_convolution_verification");
}

// McCormick bounds of a dot product on fp32 MFMA: the straight-line tiled kernel.
//
// Arithmetic and tiling are those of dot_w in dot.hip (Transformer_Verification_Code/Verifiers/Bounds.py:710-823:
// six MFMA products per K-pair into four accumulators, 128 x 64 tiles of one (head, perturbation coordinate),
// four wavefronts of 64 x 32, K-step 8, two workgroups per CU, the same order of summation: the results are the
// same bits).  What differs is everything around the MFMAs, which for a reduction of 32 ... 128 is a large part
// of a tile:
//
//   * The reduction length is a template argument (NK K-steps of 8) and a tile is straight-line code.  The first
//     MFMA of each accumulator takes the constant 0 as its addend, so no register is cleared (128 moves per tile
//     and wavefront before), and with an even NK the LDS stage of every step is known at compile time, so every
//     LDS address is an immediate.
//   * x_lw and x_uw, which need no arithmetic, go from global memory to LDS without passing through registers
//     (buffer loads with the LDS bit: a wavefront moves 1 KB per instruction, lane i's 16 bytes land at base + 16 i;
//     the swizzle of the tile is in the global address a lane asks for).  The intervals are split by sign and
//     y_lw +- y_uw formed by the staging threads as before, evenly over the four wavefronts.
//   * Every array is addressed through ONE buffer descriptor and 32-bit offsets; a tile's offsets are a handful
//     of scalar multiplies (250 scalar instructions per tile before), a K-step adds constants.
//   * The results of a tile leave BEHIND the barrier of its last K-step: vector memory operations retire in order,
//     so a wait for loads issued behind the stores would wait for the stores' acknowledgements too.
//
// Per tile and wavefront: 384 MFMAs, about 290 other vector instructions (465 before) and 200 scalar ones (490).
#include "dot_tiled.h"

namespace {

using faith::DotTiledArgs;

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void lds_void;

constexpr int TI = 128, TJ = 64, BK = 8, NTHREADS = 256;
constexpr int XT = TI * BK, YT = TJ * BK;        // floats per operand tile
// one stage of LDS: offsets of the ten operand tiles
constexpr int XL = 0, XU = XT, BH = 2 * XT, BA = 3 * XT;
constexpr int ALP = 4 * XT, ALN = ALP + YT, AUP = ALP + 2 * YT, AUN = ALP + 3 * YT, YS = ALP + 4 * YT, YD = ALP + 5 * YT;
constexpr int STAGE = 4 * XT + 6 * YT;           // 28 KB
constexpr int CHUNK = 256;                       // floats one wavefront moves per global -> LDS instruction

__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t window(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float4 ld4(__amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(r, thread_off, uniform_off, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ float2 ld2(__amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    const uintx2 v = __builtin_amdgcn_raw_buffer_load_b64(r, thread_off, uniform_off, 0);
    return make_float2(__uint_as_float(v.x), __uint_as_float(v.y));
}
// global -> LDS, 16 bytes per lane: lane i's bytes land at dst + 16 i (dst is wave-uniform)
__device__ __forceinline__ void to_lds(__amdgpu_buffer_rsrc_t r, float *dst, unsigned thread_off, unsigned uniform_off) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void *)dst, 16, thread_off, uniform_off, 0, 0);
}
__device__ __forceinline__ void st1_nt(float v, __amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, thread_off, uniform_off, 2 /* non-temporal */);
}
// one instruction each: this file is compiled with -fno-honor-nans (see dot.hip)
__device__ __forceinline__ float pos1(float v) { return __builtin_fmaxf(v, 0.f); }
__device__ __forceinline__ float neg1(float v) { return __builtin_fminf(v, 0.f); }
__device__ __forceinline__ float4 pos4(float4 v) { return make_float4(pos1(v.x), pos1(v.y), pos1(v.z), pos1(v.w)); }
__device__ __forceinline__ float4 neg4(float4 v) { return make_float4(neg1(v.x), neg1(v.y), neg1(v.z), neg1(v.w)); }
__device__ __forceinline__ float4 abs4(float4 v) {
    return make_float4(__builtin_fabsf(v.x), __builtin_fabsf(v.y), __builtin_fabsf(v.z), __builtin_fabsf(v.w));
}
// position of 16-byte half `c` (0 / 1) of row `row` inside an [rows x 8] tile: the halves are swapped on every
// other group of four rows, which makes 16-byte stores and 16-byte fragment reads free of bank conflicts
__device__ __forceinline__ int swz(int row, int c) { return row * BK + 4 * (c ^ ((row >> 2) & 1)); }

struct Walk {
    int j, i, m, h, b;      // tile numbers in mixed radix, least significant first
};
struct Offsets {
    unsigned x, b, y, a, z; // bytes from the first element of the arrays to the tile's first element
};

// This wavefront's global -> LDS loads have landed and its LDS stores are done; then the barrier.  (The compiler
// does not wait in front of a bare s_barrier on this part, and it cannot see other wavefronts' loads.)
__device__ __forceinline__ void wait_and_barrier() {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// VP = false: scores path, y is [.., Ly, D, d] (reduction axis contiguous, like x), tiles staged [row][8] with the swizzle.
// VP = true : context path, y is the value object in its own layout [.., d, D, Ly] (reduction axis slow, j contiguous),
//             and so are its intervals [.., d, Ly]; the y-side tiles are staged [k][64].
template <bool VP, int NK>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
dot_tiled(const DotTiledArgs g) {
    static_assert(NK % 2 == 0, "the LDS stage of a K-step must not depend on the tile");
    __shared__ float sm0[STAGE];
    __shared__ float sm1[STAGE];

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wi = wv / 2, wj = wv % 2;
    const int fi = lane % 32, fh = lane / 32;

    // ---- the walk: workgroup w takes the perturbation coordinates m = w (mod 8) -- workgroups are dealt to the
    // eight XCDs round robin, so the tiles that share rows of x and y meet in one L2 -- and of those the tiles
    // w / 8, w / 8 + grid / 8, ...
    const int ti = g.Lx / TI, tj = g.Ly / TJ;
    const int m_low = (int)(blockIdx.x % 8), m_radix = g.D / 8;
    auto digits = [&](int n) {
        Walk w;
        w.j = n % tj;  n /= tj;
        w.i = n % ti;  n /= ti;
        w.m = n % m_radix;  n /= m_radix;
        w.h = n % g.heads;
        w.b = n / g.heads;
        return w;
    };
    Walk cur = digits((int)(blockIdx.x / 8));
    const Walk step = digits((int)(gridDim.x / 8));
    auto advance = [&](Walk w) {
        w.j += step.j;
        if (w.j >= tj) { w.j -= tj; w.i += 1; }
        w.i += step.i;
        if (w.i >= ti) { w.i -= ti; w.m += 1; }
        w.m += step.m;
        if (w.m >= m_radix) { w.m -= m_radix; w.h += 1; }
        w.h += step.h;
        if (w.h >= g.heads) { w.h -= g.heads; w.b += 1; }
        w.b += step.b;
        return w;
    };
    int tiles_left = ((int)blockIdx.x < g.total_tiles) ? (g.total_tiles - 1 - (int)blockIdx.x) / (int)gridDim.x + 1 : 0;
    if (tiles_left == 0) return;
    auto point = [&](const Walk &w) {
        const unsigned i0 = w.i * TI, j0 = w.j * TJ, m = w.m * 8 + m_low;
        Offsets o;
        o.x = (w.b * g.xw_bs + w.h * g.xw_hs + (i0 * g.D + m) * g.xp) * 4u;
        o.b = (w.b * g.xi_bs + w.h * g.xi_hs + i0 * g.xp) * 4u;
        if (VP) {
            o.y = (w.b * g.yw_bs + w.h * g.yw_hs + m * g.yp + j0) * 4u;
            o.a = (w.b * g.yi_bs + w.h * g.yi_hs + j0) * 4u;
        } else {
            o.y = (w.b * g.yw_bs + w.h * g.yw_hs + (j0 * g.D + m) * g.yp) * 4u;
            o.a = (w.b * g.yi_bs + w.h * g.yi_hs + j0 * g.yp) * 4u;
        }
        o.z = (w.b * g.zw_bs + w.h * g.zw_hs + (i0 * g.D + m) * g.zp + j0) * 4u;
        return o;
    };
    // K-step strides in bytes
    const unsigned yk = VP ? 8u * g.D * g.yp * 4u : 32u, ak = VP ? 8u * g.yp * 4u : 32u;

    // ---- what this thread asks for, in bytes from a tile's first element (never changes)
    // global -> LDS: wavefront wv moves rows 32 wv ... 32 wv + 31 of the x-side tiles; lane i fills 16 bytes at
    // 16 i of the chunk, i.e. slot i % 2 of row i / 2, which holds half (i % 2) ^ ((row >> 2) & 1) of that row
    const int xr = 32 * wv + lane / 2, xh = (lane % 2) ^ ((xr >> 2) & 1);
    const unsigned vx = ((unsigned)xr * g.D * g.xp + xh * 4) * 4u;
    // through registers: 8 bytes of y_lw and of y_uw per thread
    unsigned vy;
    int ydst;
    if (VP) {
        const int k = tid / 32, j2 = (tid % 32) * 2;
        vy = ((unsigned)k * g.D * g.yp + j2) * 4u;
        ydst = k * TJ + j2;
    } else {
        const int row = tid / 4, q = tid % 4;
        vy = ((unsigned)row * g.D * g.yp + q * 2) * 4u;
        ydst = swz(row, q / 2) + (q % 2) * 2;
    }
    // 16 bytes of b per thread, and 16 bytes of a_l (wavefronts 0, 1) or a_u (wavefronts 2, 3)
    const int srow = tid / 2, sc = tid % 2, t2 = tid % 128;
    const unsigned vbs = ((unsigned)srow * g.xp + sc * 4) * 4u;
    const int bdst = swz(srow, sc);
    const unsigned vas = VP ? ((unsigned)(t2 / 16) * g.yp + (t2 % 16) * 4) * 4u : ((unsigned)(t2 / 2) * g.yp + (t2 % 2) * 4) * 4u;
    const int adst = VP ? (t2 / 16) * TJ + (t2 % 16) * 4 : swz(t2 / 2, t2 % 2);
    const bool upper = wv >= 2;

    const __amdgpu_buffer_rsrc_t rxl = window(g.xlw, g.x_bytes), rxu = window(g.xuw, g.x_bytes);
    const __amdgpu_buffer_rsrc_t ryl = window(g.ylw, g.y_bytes), ryu = window(g.yuw, g.y_bytes);
    const __amdgpu_buffer_rsrc_t rb = window(g.x_l, g.xi_bytes);
    const __amdgpu_buffer_rsrc_t ra = window(upper ? g.y_u : g.y_l, g.yi_bytes);      // the interval this wavefront splits
    const __amdgpu_buffer_rsrc_t rzl = window(g.zlw, g.z_bytes), rzu = window(g.zuw, g.z_bytes);

    float2 py0, py1;
    float4 pb, pa;
    // the loads of K-step kt of the tile at `o`, into stage s
    auto issue = [&](int kt, const Offsets &o, float *s) {
        const unsigned kx = kt * 32u;
        to_lds(rxl, s + XL + wv * CHUNK, vx, o.x + kx);
        to_lds(rxu, s + XU + wv * CHUNK, vx, o.x + kx);
        pb = ld4(rb, vbs, o.b + kx);
        pa = ld4(ra, vas, o.a + kt * ak);
        py0 = ld2(ryl, vy, o.y + kt * yk);
        py1 = ld2(ryu, vy, o.y + kt * yk);
    };
    // what came through registers -> stage s
    auto stage = [&](float *s) {
        *reinterpret_cast<float2 *>(s + YS + ydst) = make_float2(py0.x + py1.x, py0.y + py1.y);
        *reinterpret_cast<float2 *>(s + YD + ydst) = make_float2(py0.x - py1.x, py0.y - py1.y);
        *reinterpret_cast<float4 *>(s + BH + bdst) = pb;                      // b and |b|: P and Q come out doubled
        *reinterpret_cast<float4 *>(s + BA + bdst) = abs4(pb);               // and are halved once per result
        *reinterpret_cast<float4 *>(s + (upper ? AUP : ALP) + adst) = pos4(pa);
        *reinterpret_cast<float4 *>(s + (upper ? AUN : ALN) + adst) = neg4(pa);
    };

    // ---- fragments: x side rows wi*64 + {0, 32} + fi, y side column wj*32 + fi; this lane's four K values are
    // half `fh` of the K-step
    int fa[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) fa[s] = swz(wi * 64 + s * 32 + fi, fh);
    const int fy = VP ? (4 * fh) * TJ + wj * 32 + fi : swz(wj * 32 + fi, fh);
    auto yfrag = [&](const float *s, int o) -> float4 {
        if (VP) {
            const float *p = s + o + fy;
            return make_float4(p[0], p[TJ], p[2 * TJ], p[3 * TJ]);
        }
        return *reinterpret_cast<const float4 *>(s + o + fy);
    };

    // ---- results: z[.., i, m, j]; register r of block a is row a*32 + 8*(r/4) + 4*(lane/32) + r%4 of the wavefront
    // tile, lanes run along j.  A row is a uniform offset from the tile's first element.
    const unsigned rsb = (unsigned)g.D * g.zp * 4u;                      // one step in i, bytes
    const unsigned lane_off = (unsigned)(wi * 64 + 4 * fh) * rsb + (wj * 32 + fi) * 4u;

    Offsets here = point(cur);
    issue(0, here, sm0);
    stage(sm0);
    wait_and_barrier();

    for (; tiles_left > 0; --tiles_left) {
        const bool has_next = tiles_left > 1;
        floatx16 cl[2], cu[2], cp[2], cq[2];               // the x terms of z_lw and z_uw; P and Q of the y terms
        Offsets next = here;
#pragma unroll
        for (int kt = 0; kt < NK; ++kt) {
            float *sc_ = (kt & 1) ? sm1 : sm0, *sn_ = (kt & 1) ? sm0 : sm1;
            // the fetch of the next K-step -- the first one of the next tile included -- goes first
            if (kt < NK - 1) {
                issue(kt + 1, here, sn_);
            } else if (has_next) {
                cur = advance(cur);
                next = point(cur);
                issue(0, next, sn_);
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                const float *s = sc_;
                float4 xl[2], xu[2], bh[2], ba[2];
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    xl[a] = *reinterpret_cast<const float4 *>(s + XL + fa[a]);
                    xu[a] = *reinterpret_cast<const float4 *>(s + XU + fa[a]);
                }
                const float4 alp = yfrag(s, ALP), aup = yfrag(s, AUP), aln = yfrag(s, ALN), aun = yfrag(s, AUN);
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    bh[a] = *reinterpret_cast<const float4 *>(s + BH + fa[a]);
                    ba[a] = *reinterpret_cast<const float4 *>(s + BA + fa[a]);
                }
                const float4 ys = yfrag(s, YS), yd = yfrag(s, YD);
                if (kt == 0) {
                    // the first product of each accumulator adds to the constant 0: nothing is cleared
                    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
                        cl[a] = mfma(xl[a].x, alp.x, zero);
                        cu[a] = mfma(xu[a].x, aup.x, zero);
                    }
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
                        cl[a] = mfma(xu[a].x, aln.x, cl[a]);
                        cu[a] = mfma(xl[a].x, aun.x, cu[a]);
                    }
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
                        cp[a] = mfma(bh[a].x, ys.x, zero);
                        cq[a] = mfma(ba[a].x, yd.x, zero);
                    }
                }
#define FAITH_DOT_STEP(c)                                   \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cl[a] = mfma(xl[a].c, alp.c, cl[a]);                \
        cu[a] = mfma(xu[a].c, aup.c, cu[a]);                \
    }                                                       \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cl[a] = mfma(xu[a].c, aln.c, cl[a]);                \
        cu[a] = mfma(xl[a].c, aun.c, cu[a]);                \
    }                                                       \
    _Pragma("unroll") for (int a = 0; a < 2; ++a) {         \
        cp[a] = mfma(bh[a].c, ys.c, cp[a]);                 \
        cq[a] = mfma(ba[a].c, yd.c, cq[a]);                 \
    }
                if (kt != 0) { FAITH_DOT_STEP(x) }
                FAITH_DOT_STEP(y)
                FAITH_DOT_STEP(z)
                FAITH_DOT_STEP(w)
#undef FAITH_DOT_STEP
            }
            __builtin_amdgcn_sched_barrier(0);
            if (kt == NK - 1) {
                // The operands of the next tile's first step are staged and the barrier is passed BEFORE the results
                // leave: vector memory operations retire in order, so a wait for loads that were issued behind the
                // stores would wait for the stores' acknowledgements as well; this way the stores have a whole K-step
                // before anything waits behind them.
                if (has_next) stage(sn_);
                wait_and_barrier();
                // z_lw = X_l + (P + Q), z_uw = X_u + (P - Q); 64 stores in one run: the CU's other workgroup, which is
                // somewhere else in its own tile, has the MFMA pipe meanwhile
                unsigned step_b = rsb, z0 = here.z;
                asm volatile("" : "+s"(step_b), "+s"(z0));         // keeps 32 row offsets from being hoisted and held
#pragma unroll
                for (int a = 0; a < 2; ++a)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int row_in_tile = a * 32 + 8 * (r / 4) + r % 4;
                        const float p = cp[a][r], q = cq[a][r];
                        st1_nt(cl[a][r] + 0.5f * (p + q), rzl, lane_off, z0 + row_in_tile * step_b);
                        st1_nt(cu[a][r] + 0.5f * (p - q), rzu, lane_off, z0 + row_in_tile * step_b);
                    }
                here = next;
                __builtin_amdgcn_sched_barrier(0);
            } else {
                stage(sn_);
                wait_and_barrier();
            }
        }
    }
}

template <bool VP>
void launch_vp(int reduction, const DotTiledArgs &a, int grid, hipStream_t st) {
    if (reduction == 32)
        hipLaunchKernelGGL((dot_tiled<VP, 4>), dim3((unsigned)grid), dim3(NTHREADS), 0, st, a);
    else if (reduction == 64)
        hipLaunchKernelGGL((dot_tiled<VP, 8>), dim3((unsigned)grid), dim3(NTHREADS), 0, st, a);
    else
        hipLaunchKernelGGL((dot_tiled<VP, 16>), dim3((unsigned)grid), dim3(NTHREADS), 0, st, a);
}

}  // namespace

namespace faith {

void dot_tiled_launch(bool vp, int reduction, const DotTiledArgs &a, int grid, hipStream_t stream) {
    if (vp) launch_vp<true>(reduction, a, grid, stream);
    else launch_vp<false>(reduction, a, grid, stream);
}

}  // namespace faith

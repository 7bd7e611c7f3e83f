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
// i.e. eight products per K-pair as written.  The four y terms share their multiplier b (the planes take
// b = l_x on both sides), and b+ + b- = b, b+ - b- = |b|, so
//     sum_k b+ ylw + b- yuw = P + Q,     sum_k b+ yuw + b- ylw = P - Q,
//     P = sum_k (b/2) (ylw + yuw),       Q = sum_k (|b|/2) (ylw - yuw)
// (accumulated as 2 P and 2 Q from b and |b| and halved once per result: exact either way):
// two products where there were four -- SIX MFMA products per K-pair into four accumulators (the x terms
// of z_lw and of z_uw, P, Q), combined when a tile is done: a quarter of the MFMA time gone.  The halving
// is exact; ylw + yuw and ylw - yuw are rounded once each, by the thread that stages them.  Rows (i) come
// from x and b, columns (j) from a and y, so the accumulator tile is already laid out as z[i, m, j..]:
// lanes run along j and every store is a 128-byte run.  Neither the [Lx, D, d, Ly] broadcast the PyTorch
// code materialises nor the transposed add of its y-terms exists here.
//
// Tiling: workgroup = 4 wavefronts on a 128 x 64 (i x j) tile of one (head, m); wavefront tile
// 64 x 32 (two v_mfma_f32_32x32x2_f32 blocks along i, for each of the four accumulators).  K-step 8:
// operand tiles xlw, xuw, b, |b| [128 x 8] and a_l+, a_l-, a_u+, a_u-, ylw + yuw, ylw - yuw [64 x 8]
// = 28 KB, double buffered, two workgroups per CU.  Rows are 8 floats with the two 16-byte halves swapped
// on every other group of four rows, which makes both the 16-byte stores and the 16-byte fragment
// reads bank-conflict free without padding.
//
// On this part every vector-ALU instruction a wavefront issues takes its slot from the MFMA pipe
// (measured: 48 v_max / v_min per 64 MFMAs cost 5 % of the MFMA rate, more when interleaved), so
// the K-loop is written to issue almost none:
//   * a is split by sign, b halved and the y pair summed ONCE, by the thread that stages them, not by
//     every wavefront that reads them;
//   * global addresses are a wave-uniform 64-bit base (scalar ALU) plus a per-thread 32-bit offset
//     that only changes from tile to tile; the K-step advances the scalar base;
//   * tiles are numbered in mixed radix and walked with scalar adds and carries (no division);
//   * bounds predicates exist only on the paths for ragged tiles and a ragged last K-step.
//
// The four accumulators fill the registers two wavefronts per SIMD leave (128 of 256), so a finished
// tile is combined and stored in one run of 64 stores before the next one starts; the CU's other workgroup,
// which is somewhere else in its own tile, has the MFMA pipe meanwhile.  (With eight products and two
// accumulators a second register set let a finished tile leave piecewise under the next one's MFMAs:
// 164 us on configuration 3, against 144 us this way.)
//
// The constant terms z_lb / z_ub ([Lx, Ly] per head, 1/D_in of the work, O(1) cancelling terms)
// are summed in double by a small kernel.
#include <mutex>

#include "common.h"
#include "dot_tiled.h"
#include "dot_transposed.h"

namespace {


typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TI = 128, TJ = 64, BK = 8;
constexpr int NTHREADS = 256;
constexpr int XT = TI * BK, YT = TJ * BK;        // floats per operand tile
// one stage of LDS: offsets of the ten operand tiles
constexpr int XL = 0, XU = XT, BH = 2 * XT, BA = 3 * XT;
constexpr int ALP = 4 * XT, ALN = ALP + YT, AUP = ALP + 2 * YT, AUN = ALP + 3 * YT, YS = ALP + 4 * YT, YD = ALP + 5 * YT;
constexpr int STAGE = 4 * XT + 6 * YT;

struct DotArgs {
    const float *xlw, *xuw, *ylw, *yuw;   // [B, Lx, D, d], [B, Ly, D, d]
    const float *xlb, *xub, *ylb, *yub;   // [B, Lx, d], [B, Ly, d]
    const float *x_l, *y_l, *y_u;         // concrete intervals: b = x_l, a_l = y_l, a_u = y_u
    float *zlw, *zuw;                     // [B, Lx, D, Ly]
    float *zlb, *zub;                     // [B, Lx, Ly]
    int B, Lx, Ly, D, d;
    // Addressing of the three bound objects.  B counts (batch element, head) pairs t = b * heads + h.
    // An object either stacks them on its first axis ([B, L, D, width]: `heads` = 1 below, so that
    // b = t and h = 0) or keeps the heads of a batch element side by side in its rows
    // ([batch, L, D, heads * width], what the dense layers produce and consume).
    struct Obj {
        int pitch;      // floats from one row to the next
        int heads;      // heads side by side in a row (1: stacked)
        int width;      // floats of one head in a row
    } ox, oy, oz;
    int heads;                            // heads per batch element
    int side_by_side;                     // HEADS_X | HEADS_Y | HEADS_Z: which objects keep their heads side by side
    // Context path with a value object whose coefficients vanish outside yP key positions per batch element:
    // ylw, yuw then hold those rows only, [batch, yP, D, row of y], and y_positions [batch, yP] says which they are
    // (a value outside 0 ... d-1: no such row).  nullptr: the ordinary object.
    const long long *y_positions;
    int yP;
};
// first coefficient / first constant term of pair t of an object with `rows` positions per batch element
__device__ __forceinline__ size_t w_base(const DotArgs::Obj &o, int t, int rows, int D) {
    const int b = t / o.heads, h = t - b * o.heads;
    return (size_t)b * rows * D * o.pitch + (size_t)h * o.width;
}
__device__ __forceinline__ size_t b_base(const DotArgs::Obj &o, int t, int rows) {
    const int b = t / o.heads, h = t - b * o.heads;
    return (size_t)b * rows * o.pitch + (size_t)h * o.width;
}
constexpr int HEADS_X = 1, HEADS_Y = 2, HEADS_Z = 4;

__device__ __forceinline__ floatx16 mfma(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
// Buffer addressing keeps the three parts of an address apart in the instruction itself: a
// wave-uniform descriptor (base pointer, size), a wave-uniform 32-bit offset and a per-thread
// 32-bit offset.  With flat pointers the compiler folds the K advance into 64-bit vector adds.
// Accesses at or beyond `bytes` from the base are dropped by the hardware (loads return zero).
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ unsigned clamp32(size_t bytes) { return (bytes >> 32) ? 0xffffffffu : (unsigned)bytes; }
__device__ __forceinline__ __amdgpu_buffer_rsrc_t window(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float4 ld4(__amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    const uintx4 v = __builtin_amdgcn_raw_buffer_load_b128(r, thread_off, uniform_off, 0);
    return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ void st1_nt(float v, __amdgpu_buffer_rsrc_t r, unsigned thread_off, unsigned uniform_off) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, thread_off, uniform_off, 2 /* non-temporal */);
}
// max(v, 0) / min(v, 0), one instruction each: this file is compiled with -fno-honor-nans, without which fmaxf /
// fminf (and a median of three) come with a canonicalising v_max per value.  Plain builtins: the compiler sees the
// write, so an MFMA or an LDS store that consumes the result gets the wait states it needs.  (A NaN weight or
// interval, which the reference would carry through, is not preserved by the split.)
__device__ __forceinline__ float pos1(float v) { return __builtin_fmaxf(v, 0.f); }
__device__ __forceinline__ float neg1(float v) { return __builtin_fminf(v, 0.f); }
__device__ __forceinline__ float4 pos4(float4 v) { return make_float4(pos1(v.x), pos1(v.y), pos1(v.z), pos1(v.w)); }
__device__ __forceinline__ float4 neg4(float4 v) { return make_float4(neg1(v.x), neg1(v.y), neg1(v.z), neg1(v.w)); }
__device__ __forceinline__ float4 abs4(float4 v) {
    return make_float4(__builtin_fabsf(v.x), __builtin_fabsf(v.y), __builtin_fabsf(v.z), __builtin_fabsf(v.w));
}
__device__ __forceinline__ float4 add4(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
__device__ __forceinline__ float4 sub4(float4 a, float4 b) { return make_float4(a.x - b.x, a.y - b.y, a.z - b.z, a.w - b.w); }

// position of 16-byte half `c` (0 / 1) of row `row` inside an [rows x 8] tile
__device__ __forceinline__ int swz(int row, int c) { return row * BK + 4 * (c ^ ((row >> 2) & 1)); }

// Tile numbers in mixed radix (j-tile, i-tile, m or m / 8, head), least significant first.
struct Walk {
    int j, i, m, t;
};

// Persistent: the grid is sized to the machine (two workgroups per CU) and every workgroup walks
// tiles pid, pid + grid, ...  The walk is ONE software pipeline over (tile, K-step): the global
// loads of the next step -- the first K-step of the next tile included -- are issued before the
// MFMAs of the current step, so the head of a tile does not leave the MFMA pipe idle.
//
// xcd_map != 0 (needs dim_in % 8 == 0 and grid % 8 == 0): workgroups are dealt to the eight XCDs
// round robin, so workgroup w only takes perturbation coordinates m = w (mod 8); the tiles of one
// (head, m) -- which read the same x rows and y rows -- are then consecutive tiles of ONE XCD and
// meet in its L2.
//
// VP = false: scores path, y is [B, Ly, D, d] (reduction axis contiguous, like x).
// VP = true : context path (probs . value): y is the value bound object in its own natural layout
//   [B, d, D, Ly] -- the reduction axis (key position) is the slow one and j is contiguous --
//   and so are its concrete bounds [B, d, Ly].  The y-side tiles are then staged as [k][j]
//   (16-byte loads along j, conflict-free) and their fragments read with four 4-byte LDS reads.
//
//
// EXACT = true: d % 8 == 0, Lx % 128 == 0 and Ly % 64 == 0, so no access needs a predicate and a
// K-step is straight-line code.  EXACT = false: when d % 8 == 4, half of the last K-step lies past
// d; threads past d then read their K-step-0 element instead (in bounds) and discard it before it
// reaches LDS; rows and columns of ragged tiles are stored under a per-lane predicate.
template <bool VP, bool EXACT>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
dot_w(const DotArgs g, const int total_tiles, const int xcd_map) {
    __shared__ float sm[2][STAGE];

    const int ti = (g.Lx + TI - 1) / TI, tj = (g.Ly + TJ - 1) / TJ;
    const int d = g.d;
    const int nk = (d + BK - 1) / BK;
    constexpr bool RAGGED = !EXACT;                        // the last K-step may be half empty

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = __builtin_amdgcn_readfirstlane(tid / 64);
    const int wi = wv / 2, wj = wv % 2;
    const int fi = lane % 32, fh = lane / 32;

    // ---- the walk: this workgroup's first tile and the stride, digit by digit
    const int m_low = xcd_map ? (int)(blockIdx.x % 8) : 0;
    const int m_radix = xcd_map ? g.D / 8 : g.D;
    auto digits = [&](int n) {
        Walk w;
        w.j = n % tj;  n /= tj;
        w.i = n % ti;  n /= ti;
        w.m = n % m_radix;
        w.t = n / m_radix;
        return w;
    };
    Walk cur = digits(xcd_map ? blockIdx.x / 8 : blockIdx.x);
    const Walk step = digits(xcd_map ? gridDim.x / 8 : gridDim.x);
    auto advance = [&](Walk w) {
        w.j += step.j;
        if (w.j >= tj) { w.j -= tj; w.i += 1; }
        w.i += step.i;
        if (w.i >= ti) { w.i -= ti; w.m += 1; }
        w.m += step.m;
        if (w.m >= m_radix) { w.m -= m_radix; w.t += 1; }
        w.t += step.t;
        return w;
    };
    int tiles_left = ((int)blockIdx.x < total_tiles) ? (total_tiles - 1 - (int)blockIdx.x) / (int)gridDim.x + 1 : 0;
    if (tiles_left == 0) return;

    // ---- staging: per K-step every thread moves one float4 of xlw, xuw, b and two of the y side:
    // wavefronts 0, 1 take (a_l, a_u), wavefronts 2, 3 take (ylw, yuw)
    const int srow = tid / 2, sc = tid % 2;
    const int sdst = swz(srow, sc);
    const bool wside = wv >= 2;
    const int t2 = tid % 128;
    const int yrow = t2 / 2, yc = t2 % 2;                  // scores path: (row, half) of a y-side tile
    const int vk = t2 / 16, vj = (t2 % 16) * 4;            // context path: (k, j..j+3)
    const int ydst = VP ? vk * TJ + vj : swz(yrow, yc);
    // wave-uniform bases of the tile being loaded (bytes) and this thread's offsets from them
    const float *bxl = nullptr, *bxu = nullptr, *bbt = nullptr, *by0 = nullptr, *by1 = nullptr;
    unsigned nx = 0, nbt = 0, ny = 0;                      // bytes from those bases to the end of the tensors (< 4 GB kept)
    unsigned vx = 0, vbt = 0, vy = 0;
    // K-step strides in bytes: x side and scores-path y side advance along the contiguous axis (the
    // entry point checks that one head of y spans less than 4 GB)
    const unsigned ystride = VP ? (unsigned)BK * g.oy.pitch * (wside ? g.D : 1) * 4u : BK * 4u;
    // totals in elements
    const size_t tot_x = (size_t)g.B * g.Lx * g.D * d, tot_bt = (size_t)g.B * g.Lx * d;
    const size_t tot_y = (size_t)g.B * g.Ly * d * (wside ? g.D : 1), tot_z = (size_t)g.B * g.Lx * g.D * g.Ly;
    // results: first element of the tile being loaded (zn) and of the tile being computed (zc)
    size_t zn = 0, zc = 0;
    int zn_i0 = 0, zn_j0 = 0, zc_i0 = 0, zc_j0 = 0;
    float4 pre[5];

    auto point_at = [&](const Walk &w) {
        const int j0 = w.j * TJ, i0 = w.i * TI, t = w.t;
        const int m = xcd_map ? w.m * 8 + m_low : w.m;
        // the three objects' addressing is worked out again for every tile (a handful of scalar
        // instructions) instead of being held in scalar registers across the K-loop
        int sbs = g.side_by_side, heads = g.heads;
        asm volatile("" : "+s"(sbs), "+s"(heads));
        const int y_h = VP ? g.Ly : d, y_len = VP ? d : g.Ly;
        const DotArgs::Obj ox{(sbs & HEADS_X) ? heads * d : d, (sbs & HEADS_X) ? heads : 1, d};
        const DotArgs::Obj oy{(sbs & HEADS_Y) ? heads * y_h : y_h, (sbs & HEADS_Y) ? heads : 1, y_h};
        const DotArgs::Obj oz{(sbs & HEADS_Z) ? heads * g.Ly : g.Ly, (sbs & HEADS_Z) ? heads : 1, g.Ly};
        struct { int xp, yp, zp; } a{ox.pitch, oy.pitch, oz.pitch};
        const size_t x0 = w_base(ox, t, g.Lx, g.D) + ((size_t)i0 * g.D + m) * a.xp;
        const size_t bt0 = b_base(ox, t, g.Lx) + (size_t)i0 * a.xp;
        bxl = g.xlw + x0;  bxu = g.xuw + x0;  nx = clamp32((tot_x - x0) * 4);
        bbt = g.x_l + bt0;  nbt = clamp32((tot_bt - bt0) * 4);
        const int irow = min(srow, g.Lx - 1 - i0);         // clamped rows are never stored
        vx = ((unsigned)irow * g.D * a.xp + sc * 4) * 4u;
        vbt = ((unsigned)irow * a.xp + sc * 4) * 4u;
        size_t y0;
        if (VP) {
            // y[t, k, m, j] / a[t, k, j]; the j offset stays with the thread so that it can be clamped
            y0 = wside ? w_base(oy, t, y_len, g.D) + (size_t)m * a.yp : b_base(oy, t, y_len);
            const int jc = min(j0 + vj, g.Ly - 4);         // Ly % 4 == 0; clamped columns are never stored
            vy = ((unsigned)vk * a.yp * (wside ? g.D : 1) + jc) * 4u;
        } else {
            y0 = wside ? w_base(oy, t, y_len, g.D) + ((size_t)j0 * g.D + m) * a.yp : b_base(oy, t, y_len) + (size_t)j0 * a.yp;
            const int jrow = min(yrow, g.Ly - 1 - j0);
            vy = ((unsigned)jrow * a.yp * (wside ? g.D : 1) + yc * 4) * 4u;
        }
        by0 = (wside ? g.ylw : g.y_l) + y0;
        by1 = (wside ? g.yuw : g.y_u) + y0;
        ny = clamp32((tot_y - y0) * 4);
        zn = w_base(oz, t, g.Lx, g.D) + ((size_t)i0 * g.D + m) * a.zp + j0;
        zn_i0 = i0;
        zn_j0 = j0;
    };
    // scalar base + K advance, per-thread 32-bit offset
    auto x_past = [&](int kt) { return RAGGED && kt * BK + sc * 4 >= d; };
    auto y_past = [&](int kt) { return RAGGED && (VP ? kt * BK + vk >= d : kt * BK + yc * 4 >= d); };
    auto load_step = [&](int kt) {
        const __amdgpu_buffer_rsrc_t rxl = window(bxl, nx), rxu = window(bxu, nx), rbt = window(bbt, nbt);
        const __amdgpu_buffer_rsrc_t ry0 = window(by0, ny), ry1 = window(by1, ny);
        const unsigned kx = kt * (BK * 4u), ky = kt * ystride;
        if (RAGGED) {
            const unsigned ox = x_past(kt) ? 0u : kx, oy = y_past(kt) ? 0u : ky;
            pre[0] = ld4(rxl, vx + ox, 0);
            pre[1] = ld4(rxu, vx + ox, 0);
            pre[2] = ld4(rbt, vbt + ox, 0);
            pre[3] = ld4(ry0, vy + oy, 0);
            pre[4] = ld4(ry1, vy + oy, 0);
        } else {
            pre[0] = ld4(rxl, vx, kx);
            pre[1] = ld4(rxu, vx, kx);
            pre[2] = ld4(rbt, vbt, kx);
            pre[3] = ld4(ry0, vy, ky);
            pre[4] = ld4(ry1, vy, ky);
        }
    };
    // registers -> LDS stage `buf`; kt is the K-step the registers hold
    auto lstore = [&](int buf, int kt) {
        if (RAGGED) {
            const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
            if (x_past(kt)) pre[0] = pre[1] = pre[2] = zero;
            if (y_past(kt)) pre[3] = pre[4] = zero;
        }
        float *s = sm[buf];
        *reinterpret_cast<float4 *>(s + XL + sdst) = pre[0];
        *reinterpret_cast<float4 *>(s + XU + sdst) = pre[1];
        *reinterpret_cast<float4 *>(s + BH + sdst) = pre[2];                 // b and |b|: P and Q come out doubled
        *reinterpret_cast<float4 *>(s + BA + sdst) = abs4(pre[2]);          // and are halved once per result
        if (wside) {
            *reinterpret_cast<float4 *>(s + YS + ydst) = add4(pre[3], pre[4]);
            *reinterpret_cast<float4 *>(s + YD + ydst) = sub4(pre[3], pre[4]);
        } else {
            *reinterpret_cast<float4 *>(s + ALP + ydst) = pos4(pre[3]);
            *reinterpret_cast<float4 *>(s + ALN + ydst) = neg4(pre[3]);
            *reinterpret_cast<float4 *>(s + AUP + ydst) = pos4(pre[4]);
            *reinterpret_cast<float4 *>(s + AUN + ydst) = neg4(pre[4]);
        }
    };

    // ---- fragments: x side rows wi*64 + {0, 32} + fi, y side column wj*32 + fi; this lane's four K
    // values are half `fh` of the K-step
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
    floatx16 cl[2], cu[2], cp[2], cq[2];                   // the x terms of z_lw and z_uw; P and Q of the y terms
    auto compute = [&](int buf) {
        const float *s = sm[buf];
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
        FAITH_DOT_STEP(x)
        FAITH_DOT_STEP(y)
        FAITH_DOT_STEP(z)
        FAITH_DOT_STEP(w)
#undef FAITH_DOT_STEP
    };

    // ---- results of a finished tile: z[t, i, m, j]; register r of block a is row
    // a*32 + 8*(r/4) + 4*(lane/32) + r%4 of the wavefront tile, lanes run along j.  A row is a uniform offset
    // from the tile's first element, the lane's own offset never changes (the entry point checks that a tile
    // spans less than 4 GB).  z_lw = X_l + (P + Q), z_uw = X_u + (P - Q).  The 64 stores leave in one run: the
    // wavefront's next MFMA waits for them to issue; the CU's other workgroup, which is somewhere else in
    // its own tile, has the MFMA pipe meanwhile.
    const unsigned rsb = (unsigned)g.D * g.oz.pitch * 4u;        // one step in i, bytes
    const unsigned lane_off = (unsigned)(wi * 64 + 4 * fh) * rsb + (wj * 32 + fi) * 4u;
    auto store_tile = [&]() {
        const unsigned zbytes = clamp32((tot_z - zc) * 4);
        const __amdgpu_buffer_rsrc_t rl = window(g.zlw + zc, zbytes), ru = window(g.zuw + zc, zbytes);
        // !EXACT: rows this lane may store (0: none)
        const int rows = zc_j0 + wj * 32 + fi < g.Ly ? g.Lx - (zc_i0 + wi * 64 + 4 * fh) : 0;
        unsigned step_b = rsb;
        asm volatile("" : "+s"(step_b));                   // keeps 32 row offsets from being hoisted and held
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row_in_tile = a * 32 + 8 * (r / 4) + r % 4;
                if (EXACT || row_in_tile < rows) {
                    const float p = cp[a][r], q = cq[a][r];
                    st1_nt(cl[a][r] + 0.5f * (p + q), rl, lane_off, row_in_tile * step_b);
                    st1_nt(cu[a][r] + 0.5f * (p - q), ru, lane_off, row_in_tile * step_b);
                }
            }
    };

    point_at(cur);
    load_step(0);
    lstore(0, 0);
    zc = zn;  zc_i0 = zn_i0;  zc_j0 = zn_j0;
    __syncthreads();
    int buf = 0;

    // One K-step that is not the last of its tile: fetch the next step, multiply this one, stage the fetched
    // step.  Straight-line when EXACT, so that loads and scalar work can sit between the MFMAs; the staging must
    // stay behind them (it waits for the fetch).
    auto inner_step = [&](int kt) {
        load_step(kt + 1);
        __builtin_amdgcn_sched_barrier(0);                 // the fetch goes first
        compute(buf);
        __builtin_amdgcn_sched_barrier(0);
        lstore(buf ^ 1, kt + 1);
        __syncthreads();
        buf ^= 1;
    };

    for (; tiles_left > 0; --tiles_left) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) cl[a][r] = cu[a][r] = cp[a][r] = cq[a][r] = 0.f;
        const bool has_next = tiles_left > 1;
        for (int kt = 0; kt < nk - 1; ++kt) inner_step(kt);
        // last K-step: the fetch is the first step of the next tile
        if (has_next) {
            cur = advance(cur);
            point_at(cur);
            load_step(0);
        }
        __builtin_amdgcn_sched_barrier(0);
        compute(buf);
        __builtin_amdgcn_sched_barrier(0);
        store_tile();
        zc = zn;  zc_i0 = zn_i0;  zc_j0 = zn_j0;
        if (has_next) lstore(buf ^ 1, 0);
        __syncthreads();
        buf ^= 1;
    }
}

// Constant terms (Bounds.py:761-762 gamma, :804-807, :815-818): a workgroup owns an 8 x 8 tile of
// (i, j) of one head; four groups of 64 threads each take a quarter of every 64-wide chunk of the
// reduction, the seven [8 x chunk] operand rows are staged in LDS, sums are kept in double and the
// four partial sums meet in LDS at the end.
constexpr int BT_T = 8, BT_K = 64, BT_S = 4;
constexpr int BT_LDS = 7 * BT_T * (BT_K + 1) + 2 * 2 * BT_S * BT_T * BT_T;      // floats of LDS a tile needs
template <bool VP>
__device__ __forceinline__ void dot_b_tile(const DotArgs &g, int pid, float *smem) {
    float(*sx)[BT_T][BT_K + 1] = reinterpret_cast<float(*)[BT_T][BT_K + 1]>(smem);                             // b (= l_x), xlb, xub
    float(*sy)[BT_T][BT_K + 1] = reinterpret_cast<float(*)[BT_T][BT_K + 1]>(smem + 3 * BT_T * (BT_K + 1));    // a_l, a_u, ylb, yub
    double(*red)[BT_S][BT_T * BT_T] = reinterpret_cast<double(*)[BT_S][BT_T * BT_T]>(smem + 7 * BT_T * (BT_K + 1));   // 3640 floats in: 8-byte aligned
    const int ti = (g.Lx + BT_T - 1) / BT_T, tj = (g.Ly + BT_T - 1) / BT_T;
    const int j0 = (pid % tj) * BT_T;  pid /= tj;
    const int i0 = (pid % ti) * BT_T;  pid /= ti;
    const int t = pid;
    const int ks = threadIdx.x / 64, o = threadIdx.x % 64;
    const int tx = o % BT_T, ty = o / BT_T;                     // output (i0 + ty, j0 + tx)
    double sl = 0.0, su = 0.0;
    for (int k0 = 0; k0 < g.d; k0 += BT_K) {
        for (int e = threadIdx.x; e < BT_T * BT_K; e += 256) {
            // x rows are contiguous along k; so are y rows on the scores path, while on the context path
            // y is contiguous along j
            const int r = e / BT_K, k = e % BT_K;
            const bool xin = k0 + k < g.d && i0 + r < g.Lx;
            const size_t xo = b_base(g.ox, t, g.Lx) + (size_t)(i0 + r) * g.ox.pitch + k0 + k;
            sx[0][r][k] = xin ? g.x_l[xo] : 0.f;
            sx[1][r][k] = xin ? g.xlb[xo] : 0.f;
            sx[2][r][k] = xin ? g.xub[xo] : 0.f;
            const int ry = VP ? e % BT_T : r, ky = VP ? e / BT_T : k;
            const bool yin = k0 + ky < g.d && j0 + ry < g.Ly;
            const size_t yo = b_base(g.oy, t, VP ? g.d : g.Ly) + (VP ? (size_t)(k0 + ky) * g.oy.pitch + j0 + ry : (size_t)(j0 + ry) * g.oy.pitch + k0 + ky);
            sy[0][ry][ky] = yin ? g.y_l[yo] : 0.f;
            sy[1][ry][ky] = yin ? g.y_u[yo] : 0.f;
            sy[2][ry][ky] = yin ? g.ylb[yo] : 0.f;
            sy[3][ry][ky] = yin ? g.yub[yo] : 0.f;
        }
        __syncthreads();
#pragma unroll 4
        for (int kk = 0; kk < BT_K / BT_S; ++kk) {
            const int k = ks * (BT_K / BT_S) + kk;
            const double bt = sx[0][ty][k], xlb = sx[1][ty][k], xub = sx[2][ty][k];
            const double al = sy[0][tx][k], au = sy[1][tx][k], ylb = sy[2][tx][k], yub = sy[3][tx][k];
            const double bp = bt > 0 ? bt : 0, bn = bt < 0 ? bt : 0;
            sl += -al * bt + (al > 0 ? al * xlb : al * xub) + bp * ylb + bn * yub;
            su += -au * bt + (au > 0 ? au * xub : au * xlb) + bp * yub + bn * ylb;
        }
        __syncthreads();
    }
    red[0][ks][o] = sl;
    red[1][ks][o] = su;
    __syncthreads();
    if (ks == 0) {
        const int i = i0 + ty, j = j0 + tx;
        if (i < g.Lx && j < g.Ly) {
            const size_t z = b_base(g.oz, t, g.Lx) + (size_t)i * g.oz.pitch + j;
            g.zlb[z] = (float)(red[0][0][o] + red[0][1][o] + red[0][2][o] + red[0][3][o]);
            g.zub[z] = (float)(red[1][0][o] + red[1][1][o] + red[1][2][o] + red[1][3][o]);
        }
    }
}

template <bool VP>
__global__ void __launch_bounds__(256) dot_b(const DotArgs g) {
    __shared__ __align__(16) float sm[BT_LDS];
    dot_b_tile<VP>(g, blockIdx.x, sm);
}

// Short sequences (Lx, Ly <= 64, d <= 80): the 128 x 64 tile above would be mostly padding, so here
// a WAVEFRONT owns one 32 x 32 block of z for one perturbation coordinate m (one MFMA block for
// z_lw, one for z_uw).  The four wavefronts of a workgroup share the (head, i-block, j-block): the
// operands that do not depend on m (b, |b|, a_l+-, a_u+- split by sign) are staged in LDS once for
// the whole reduction, and every wavefront walks its own `mpw` coordinates, loading its x and y
// fragments straight from global memory in MFMA layout (rows of 32 bytes per lane and K-step: poor
// coalescing, but these problems are a few megabytes and latency is what counts).
constexpr int SB = 32;                         // block edge
// The workgroups from `w_tiles` on take the 8 x 8 tiles of the constant terms instead (short chains of double
// arithmetic that run beside the MFMA blocks rather than in a launch of their own).  They come last: the
// MFMA workgroups that share rows of x count on starting together.
//
// RAGGED (context path only): the reduction length -- the number of key positions -- is any number, as the
// length of a sentence is.  The staged operands are zero beyond it, up to the next multiple of 8, so whatever
// the fragments of x and y hold there (the start of the next row, or the zero that reads past the end of a
// tensor return) does not count; the rows of x then start on any 4-byte boundary and are read 4 bytes at a time.
//
// COMPACT_Y (context path only): the value object has coefficients at a few key positions only (DotArgs::y_positions).
// Its y terms, sum_k b(i, k) y(k, m, j), then have one addend per such position: no y fragments, no P and Q
// accumulators; the addends are formed from b in LDS and the lane's column of the compact rows when the block is stored.
template <bool VP, bool RAGGED = false, bool COMPACT_Y = false>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(COMPACT_Y ? 4 : 3, COMPACT_Y ? 4 : 3)))
dot_w_small(const DotArgs g, const int mpw, const int heads_first, const int w_tiles) {
    static_assert(VP || !RAGGED, "a ragged reduction exists on the context path only");
    static_assert(VP || !COMPACT_Y, "compact value operands exist on the context path only");
    extern __shared__ __align__(16) float sh[];   // six operands, each d/8 swizzled [32 x 8] pieces (or a constant-term tile)
    if ((int)blockIdx.x >= w_tiles) {
        dot_b_tile<VP>(g, blockIdx.x - w_tiles, sh);
        return;
    }
    const int d = g.d;
    const int dp = RAGGED ? (d + 7) / 8 * 8 : d, nq = dp / 8;      // the reduction as the MFMAs walk it
    const int OP = SB * dp;                    // floats per operand
    float *s_bp = sh, *s_bn = sh + OP, *s_alp = sh + 2 * OP, *s_aln = sh + 3 * OP, *s_aup = sh + 4 * OP, *s_aun = sh + 5 * OP;

    const int nib = (g.Lx + SB - 1) / SB, njb = (g.Ly + SB - 1) / SB;
    const int mgroups = (g.D + 4 * mpw - 1) / (4 * mpw);
    // heads_first: the heads lie side by side in the rows of x, so workgroups that run together take
    // the same rows of different heads and their 32-byte pieces add up to whole rows
    int pid = blockIdx.x;
    int t = 0;
    if (heads_first) { t = pid % g.B;  pid /= g.B; }     // (batch, head) pairs fastest
    const int mg = pid % mgroups;  pid /= mgroups;
    const int j0 = (pid % njb) * SB;  pid /= njb;
    const int i0 = (pid % nib) * SB;  pid /= nib;
    if (!heads_first) t = pid;

    const int tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int fi = lane % 32, fh = lane / 32;

    // first elements of this (batch element, head) in the three objects
    const int y_len = VP ? g.d : g.Ly;
    const size_t xb0 = b_base(g.ox, t, g.Lx), yb0 = b_base(g.oy, t, y_len);
    const size_t xw0 = w_base(g.ox, t, g.Lx, g.D), yw0 = w_base(g.oy, t, y_len, g.D), zw0 = w_base(g.oz, t, g.Lx, g.D);

    // ---- operands shared by every m: b = l_x rows i0.., a_l / a_u rows (columns of z) j0..
    if (RAGGED) {
        for (int e = tid; e < SB * dp; e += 256) {
            const int row = e / dp, k = e % dp;
            const float bt = k < d ? g.x_l[xb0 + (size_t)min(i0 + row, g.Lx - 1) * g.ox.pitch + k] : 0.f;
            const int dst = (k / 8) * (SB * 8) + swz(row, (k % 8) / 4) + k % 4;
            s_bp[dst] = bt;                            // b and |b|: see the top of the file
            s_bn[dst] = __builtin_fabsf(bt);
        }
    }
    for (int e = tid; !RAGGED && e < SB * d / 4; e += 256) {
        const int row = e / (d / 4), c4 = e % (d / 4);
        const int dst = (c4 / 2) * (SB * 8) + swz(row, c4 % 2);
        const float4 bt = *reinterpret_cast<const float4 *>(g.x_l + xb0 + (size_t)min(i0 + row, g.Lx - 1) * g.ox.pitch + c4 * 4);
        *reinterpret_cast<float4 *>(s_bp + dst) = bt;                // b and |b|: see the top of the file
        *reinterpret_cast<float4 *>(s_bn + dst) = abs4(bt);
        if (!VP) {
            const size_t o = yb0 + (size_t)min(j0 + row, g.Ly - 1) * g.oy.pitch + c4 * 4;
            const float4 al = *reinterpret_cast<const float4 *>(g.y_l + o), au = *reinterpret_cast<const float4 *>(g.y_u + o);
            *reinterpret_cast<float4 *>(s_alp + dst) = pos4(al);
            *reinterpret_cast<float4 *>(s_aln + dst) = neg4(al);
            *reinterpret_cast<float4 *>(s_aup + dst) = pos4(au);
            *reinterpret_cast<float4 *>(s_aun + dst) = neg4(au);
        }
    }
    if (VP) {
        // a[t, k, j]: j is the contiguous axis
        for (int e = tid; e < SB * dp; e += 256) {
            const int j = e % SB, k = e / SB;
            const size_t o = yb0 + (size_t)min(k, d - 1) * g.oy.pitch + min(j0 + j, g.Ly - 1);
            const float al = k < d ? g.y_l[o] : 0.f, au = k < d ? g.y_u[o] : 0.f;
            const int dst = (k / 8) * (SB * 8) + swz(j, (k % 8) / 4) + k % 4;
            s_alp[dst] = pos1(al);
            s_aln[dst] = neg1(al);
            s_aup[dst] = pos1(au);
            s_aun[dst] = neg1(au);
        }
    }
    __syncthreads();

    const int frag = swz(fi, fh);              // this lane's 16 bytes inside a [32 x 8] piece
    const int irow = min(i0 + fi, g.Lx - 1), jcol = min(j0 + fi, g.Ly - 1);
    const int wave = __builtin_amdgcn_readfirstlane(wv);
    // per-lane byte offsets from the first element of (head, m); they do not depend on m
    const unsigned vx = ((unsigned)irow * g.D * g.ox.pitch + fh * 4) * 4u;
    const unsigned vy = VP ? ((unsigned)(fh * 4) * g.D * g.oy.pitch + jcol) * 4u : ((unsigned)jcol * g.D * g.oy.pitch + fh * 4) * 4u;
    const unsigned ykstep = (unsigned)g.D * g.oy.pitch * 4u;             // context path: one step in k, bytes
    const size_t tot_x = (size_t)g.B * g.Lx * g.D * d, tot_y = (size_t)g.B * g.Ly * g.D * d;
    for (int s = 0; s < mpw; ++s) {
        const int m = (mg * 4 + wave) * mpw + s;
        if (m >= g.D) break;
        // windows that start at (head t, coordinate m) and end with the tensor
        const size_t x0 = xw0 + (size_t)m * g.ox.pitch, y0 = yw0 + (size_t)m * g.oy.pitch;
        const __amdgpu_buffer_rsrc_t wxl = window(g.xlw + x0, clamp32((tot_x - x0) * 4));
        const __amdgpu_buffer_rsrc_t wxu = window(g.xuw + x0, clamp32((tot_x - x0) * 4));
        const __amdgpu_buffer_rsrc_t wyl = window(g.ylw + y0, clamp32((tot_y - y0) * 4));
        const __amdgpu_buffer_rsrc_t wyu = window(g.yuw + y0, clamp32((tot_y - y0) * 4));
        floatx16 cl, cu, cp, cq;                   // x terms of z_lw and z_uw; P and Q of the y terms
#pragma unroll
        for (int r = 0; r < 16; ++r) cl[r] = cu[r] = cp[r] = cq[r] = 0.f;
        for (int q0 = 0; q0 < nq; q0 += 4) {
            float4 xl[4], xu[4], yl[4], yu[4];
#pragma unroll
            for (int qq = 0; qq < 4; ++qq) {
                if (q0 + qq < nq) {
                    const unsigned k = (q0 + qq) * 8;
                    if (RAGGED) {
                        float xv[2][4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            xv[0][c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wxl, vx, (k + c) * 4u, 0));
                            xv[1][c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wxu, vx, (k + c) * 4u, 0));
                        }
                        xl[qq] = make_float4(xv[0][0], xv[0][1], xv[0][2], xv[0][3]);
                        xu[qq] = make_float4(xv[1][0], xv[1][1], xv[1][2], xv[1][3]);
                    } else {
                        xl[qq] = ld4(wxl, vx, k * 4u);
                        xu[qq] = ld4(wxu, vx, k * 4u);
                    }
                    if (COMPACT_Y) {
                        yl[qq] = yu[qq] = make_float4(0.f, 0.f, 0.f, 0.f);
                    } else if (VP) {
                        // y[t, k, m, j]: four keys, one column per lane
                        float yv[2][4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            yv[0][c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wyl, vy, (k + c) * ykstep, 0));
                            yv[1][c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wyu, vy, (k + c) * ykstep, 0));
                        }
                        yl[qq] = make_float4(yv[0][0], yv[0][1], yv[0][2], yv[0][3]);
                        yu[qq] = make_float4(yv[1][0], yv[1][1], yv[1][2], yv[1][3]);
                    } else {
                        yl[qq] = ld4(wyl, vy, k * 4u);
                        yu[qq] = ld4(wyu, vy, k * 4u);
                    }
                }
            }
#pragma unroll
            for (int qq = 0; qq < 4; ++qq) {
                if (q0 + qq < nq) {
                    const int o = (q0 + qq) * (SB * 8) + frag;
                    const float4 bh = *reinterpret_cast<const float4 *>(s_bp + o), ba = *reinterpret_cast<const float4 *>(s_bn + o);
                    const float4 alp = *reinterpret_cast<const float4 *>(s_alp + o), aln = *reinterpret_cast<const float4 *>(s_aln + o);
                    const float4 aup = *reinterpret_cast<const float4 *>(s_aup + o), aun = *reinterpret_cast<const float4 *>(s_aun + o);
                    const float4 ys = add4(yl[qq], yu[qq]), yd = sub4(yl[qq], yu[qq]);
#define FAITH_DOT_SMALL(c)                          \
    cl = mfma(xl[qq].c, alp.c, cl);                 \
    cu = mfma(xu[qq].c, aup.c, cu);                 \
    if (!COMPACT_Y) cp = mfma(bh.c, ys.c, cp);      \
    cl = mfma(xu[qq].c, aln.c, cl);                 \
    cu = mfma(xl[qq].c, aun.c, cu);                 \
    if (!COMPACT_Y) cq = mfma(ba.c, yd.c, cq);
                    FAITH_DOT_SMALL(x)
                    FAITH_DOT_SMALL(y)
                    FAITH_DOT_SMALL(z)
                    FAITH_DOT_SMALL(w)
#undef FAITH_DOT_SMALL
                }
            }
        }
        // register r is row 8*(r/4) + 4*(lane/32) + r%4 of the block, lanes run along j
        if (COMPACT_Y) {
            // the y terms, b+ y_lw + b- y_uw and b+ y_uw + b- y_lw, have one addend per key position that has
            // coefficients: b from the staged tile, the lane's column of the compact row; added to the x terms in place
            const int yb = t / g.oy.heads, yh = t - yb * g.oy.heads;
            for (int p = 0; p < g.yP; ++p) {
                const long long kp = g.y_positions[(size_t)yb * g.yP + p];
                if (kp < 0 || kp >= d) continue;                        // no such row (the same for every lane)
                const int kk = (int)kp;
                const size_t o = (((size_t)yb * g.yP + p) * g.D + m) * g.oy.pitch + (size_t)yh * g.oy.width + jcol;
                const float vl = g.ylw[o], vu = g.yuw[o];
                // row 8*(r/4) + 4*fh + r%4 of piece kk/8: bit 2 of the row is fh, so the swizzle is the lane's own
                const float *bsrc = s_bp + (kk / 8) * (SB * 8) + 32 * fh + 4 * (((kk % 8) / 4) ^ fh) + kk % 4;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float bt = bsrc[(8 * (r / 4) + (r % 4)) * 8];
                    const float bp = fmaxf(bt, 0.f), bn = fminf(bt, 0.f);
                    cl[r] += bp * vl + bn * vu;
                    cu[r] += bp * vu + bn * vl;
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pp = cp[r], qq_ = cq[r];
                cl[r] += 0.5f * (pp + qq_);
                cu[r] += 0.5f * (pp - qq_);
            }
        }
        // Buffer stores: the window is this block's rows of z at coordinate m (it ends behind the last row that exists),
        // a register's row is a wave-uniform offset, the lane's offset is fixed; a lane without a column is sent outside.
        {
            const size_t z0 = zw0 + ((size_t)i0 * g.D + m) * g.oz.pitch + j0;
            const unsigned row_b = (unsigned)g.D * g.oz.pitch * 4u;                 // one row i, bytes
            const int rows_here = min(SB, g.Lx - i0);
            const unsigned bytes = (unsigned)(rows_here - 1) * row_b + (unsigned)min(SB, g.Ly - j0) * 4u;   // <= rows_here * row_b
            const __amdgpu_buffer_rsrc_t wzl = window(g.zlw + z0, bytes), wzu = window(g.zuw + z0, bytes);
            const unsigned vo = j0 + fi < g.Ly ? (unsigned)(4 * fh) * row_b + (unsigned)fi * 4u : 0x80000000u;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const unsigned so = (unsigned)(8 * (r / 4) + (r % 4)) * row_b;
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(cl[r]), wzl, vo, so, 2 /* non-temporal */);
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(cu[r]), wzu, vo, so, 2);
            }
        }
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
        const float *xl = g.xlw + w_base(g.ox, t, g.Lx, g.D) + ((size_t)i * g.D + m) * g.ox.pitch;
        const float *xu = g.xuw + w_base(g.ox, t, g.Lx, g.D) + ((size_t)i * g.D + m) * g.ox.pitch;
        // y element (j, m, k): scores path [t, j, m, k]; context path [t, k, m, j]
        const size_t ybase = w_base(g.oy, t, VP ? g.d : g.Ly, g.D) + (VP ? (size_t)m * g.oy.pitch + j : ((size_t)j * g.D + m) * g.oy.pitch);
        const size_t ystep = VP ? (size_t)g.D * g.oy.pitch : 1;
        const size_t abase = b_base(g.oy, t, VP ? g.d : g.Ly) + (VP ? (size_t)j : (size_t)j * g.oy.pitch);
        const size_t astep = VP ? g.oy.pitch : 1;
        const float *bt = g.x_l + b_base(g.ox, t, g.Lx) + (size_t)i * g.ox.pitch;
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
        const size_t z = w_base(g.oz, t, g.Lx, g.D) + ((size_t)i * g.D + m) * g.oz.pitch + j;
        g.zlw[z] = (float)sl;
        g.zuw[z] = (float)su;
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
    const size_t xo = b_base(g.ox, t, g.Lx) + (size_t)i * g.ox.pitch;
    const size_t yo = b_base(g.oy, t, VP ? g.d : g.Ly) + (VP ? (size_t)j : (size_t)j * g.oy.pitch), ys = VP ? g.oy.pitch : 1;
    float lo = 0.f, hi = 0.f;
    for (int k = 0; k < g.d; ++k) {
        const float l1 = g.xlb[xo + k], u1 = g.xub[xo + k], l2 = g.ylb[yo + k * ys], u2 = g.yub[yo + k * ys];
        const float c1 = l1 * l2, c2 = l1 * u2, c3 = u1 * l2, c4 = u1 * u2;
        lo += fminf(fminf(c1, c2), fminf(c3, c4));
        hi += fmaxf(fmaxf(c1, c2), fmaxf(c3, c4));
    }
    const size_t zb = b_base(g.oz, t, g.Lx) + (size_t)i * g.oz.pitch + j, zw = w_base(g.oz, t, g.Lx, g.D) + (size_t)i * g.oz.pitch + j;   // dim_in == 1
    g.zlb[zb] = lo;
    g.zub[zb] = hi;
    g.zlw[zw] = 0.f;
    g.zuw[zw] = 0.f;
}

// Shared body of the two entry points.  For the context path (VP) `d` is the number of key positions
// (the reduction length) and `Ly` the width of the value vectors; y_* are the value bounds in their
// natural layout [B, d, D, Ly] / [B, d, Ly].
//
// `side_by_side` says which of the bound objects keep their heads side by side in the rows of one
// object [1, L, D, heads * width] instead of stacked on the batch axis (HEADS_X / HEADS_Y / HEADS_Z);
// the concrete intervals of such an object have that layout too.
template <bool VP>
int dot_entry(const char *who, float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb, const float *x_ub,
              const float *y_lb, const float *y_ub, const float *x_lw, const float *x_uw, const float *y_lw,
              const float *y_uw, float *z_lb, float *z_ub, float *z_lw, float *z_uw, int B, int Lx, int Ly, int d, int D,
              float epsilon, int q, int words, int side_by_side, int heads, void *stream,
              const long long *y_positions = nullptr, int y_n_positions = 0) {
    // y_positions (context path): y_lw, y_uw hold the coefficient rows of those key positions only, and y_l, y_u are
    // given (the caller concretized the rows that exist); only the per-wavefront kernel takes such an operand
    const bool compact_y = y_positions != nullptr;
    FAITH_NOT_NULL(x_l); FAITH_NOT_NULL(y_l); FAITH_NOT_NULL(y_u);      // x_u may be NULL: not wanted
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub);
    FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_NOT_NULL(z_lb); FAITH_NOT_NULL(z_ub); FAITH_NOT_NULL(z_lw); FAITH_NOT_NULL(z_uw);
    FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_ALIGNED4(z_lw); FAITH_ALIGNED4(z_uw); FAITH_ALIGNED4(z_lb); FAITH_ALIGNED4(z_ub);
    FAITH_REQUIRE(B > 0 && Lx > 0 && Ly > 0 && d > 0 && D > 0, FAITH_ERR_SHAPE,
                  "%s: batch=%d rows of x=%d columns of z=%d reduction length=%d dim_in=%d must be positive", who, B,
                  Lx, Ly, d, D);
    const long long nw = (long long)B * Lx * D * Ly;
    FAITH_REQUIRE((long long)B * (Lx > Ly ? Lx : Ly) * D <= 0x7fffffffLL && (long long)B * d * D <= 0x7fffffffLL,
                  FAITH_ERR_SHAPE, "%s: batch*length*dim_in exceeds 2^31", who);

    hipStream_t st = static_cast<hipStream_t>(stream);
    DotArgs g{x_lw, x_uw, y_lw, y_uw, x_lb, x_ub, y_lb, y_ub, x_l, y_l, y_u, z_lw, z_uw, z_lb, z_ub, B, Lx, Ly, D, d};
    // y is [rows of y, D, width of y] per head
    const int y_len = VP ? d : Ly, y_h = VP ? Ly : d;
    const bool x_sbs = side_by_side & HEADS_X, y_sbs = side_by_side & HEADS_Y, z_sbs = side_by_side & HEADS_Z;
    FAITH_REQUIRE(heads >= 1 && B % heads == 0, FAITH_ERR_SHAPE, "%s: %d heads do not divide %d (batch, head) pairs", who,
                  heads, B);
    FAITH_REQUIRE((long long)heads * (d > Ly ? d : Ly) <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: heads * row width exceeds 2^31", who);
    g.ox = {x_sbs ? heads * d : d, x_sbs ? heads : 1, d};
    g.oy = {y_sbs ? heads * y_h : y_h, y_sbs ? heads : 1, y_h};
    g.oz = {z_sbs ? heads * Ly : Ly, z_sbs ? heads : 1, Ly};
    g.heads = heads;
    g.side_by_side = side_by_side;
    g.y_positions = y_positions;
    g.yP = y_n_positions;
    FAITH_REQUIRE(!compact_y || (VP && y_n_positions > 0 && D > 1 && ((uintptr_t)y_positions & 7) == 0 &&
                                 (long long)(B / heads) * y_n_positions * D <= 0x7fffffffLL), FAITH_ERR_UNSUPPORTED,
                  "%s: a compact value operand needs the context path, dim_in > 1 and at least one position", who);
    FAITH_REQUIRE(words >= 1 && (D == 1 || D % words == 0), FAITH_ERR_SHAPE, "%s: words=%d must divide dim_in=%d", who, words, D);
    // concrete intervals of both operands (Bounds.py:725-726); x_u is produced because the reference
    // interface exposes it, the planes do not use it.  One launch for both objects.
    // An object with its heads side by side is concretized as the one [L, D, heads * width] object it is.
    // (With dim_in == 1 the interval shortcut below does not read them; they are still the documented
    // outputs of the entry point, so they are written there too.)
    const int cx_rows = x_sbs ? B / heads * Lx : B * Lx, cx_h = x_sbs ? heads * d : d;
    const int cy_rows = y_sbs ? B / heads * y_len : B * y_len, cy_h = y_sbs ? heads * y_h : y_h;
    // dim_in == 1 with several words: the reference's blocks are then empty (dim_in // words == 0,
    // Bounds.py:319-326) and its intervals are the constant terms themselves -- a radius of zero here
    const bool empty_blocks = D == 1 && words > 1;
    int rc = faith::concretize_pair(x_lb, x_ub, x_lw, x_uw, x_l, x_u, cx_rows, y_lb, y_ub, y_lw, y_uw, y_l, y_u,
                                    compact_y ? 0 : cy_rows, D, cx_h, cy_h, empty_blocks ? 0.f : epsilon, q,
                                    empty_blocks ? 1 : words, stream);
    if (rc != FAITH_OK) return rc;
    if (D == 1) {
        const long long n = (long long)B * Lx * Ly;
        hipLaunchKernelGGL(dot_interval<VP>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, g);
        return faith::check_launch(who);
    }

    const long long b_tiles = (long long)B * ((Lx + BT_T - 1) / BT_T) * ((Ly + BT_T - 1) / BT_T);
    FAITH_REQUIRE(b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
    auto constant_terms = [&]() { hipLaunchKernelGGL(dot_b<VP>, dim3((unsigned)b_tiles), dim3(256), 0, st, g); };

    const int max_pitch = g.ox.pitch > g.oy.pitch ? (g.ox.pitch > g.oz.pitch ? g.ox.pitch : g.oz.pitch) : (g.oy.pitch > g.oz.pitch ? g.oy.pitch : g.oz.pitch);
    const bool fast = (d % 4 == 0) && (!VP || Ly % 4 == 0) && faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) &&
                      faith::aligned(y_lw, 16) && faith::aligned(y_uw, 16) && faith::aligned(x_l, 16) &&
                      faith::aligned(y_l, 16) && faith::aligned(y_u, 16) &&
                      (long long)TI * D * max_pitch * 4 < 0xffffffffLL &&            // 32-bit offsets inside a tile
                      (!VP || (long long)d * D * g.oy.pitch * 4 < 0xffffffffLL);           // and along K inside a head
    // The per-wavefront kernel runs at about 0.85 of the tiled kernel's rate on the same padded work, so it
    // takes the problems whose 32 x 32 blocks cover at most 0.85 of what 128 x 64 tiles would (sequence
    // lengths up to 64, and e.g. 80 ... 112: 119 against 164 us at 4 heads, L = 80).  The tuning knob can
    // force either kernel.
    const bool small_ok = fast && d % 8 == 0 && d <= 80;
    const int pick = faith::tune_get(FAITH_TUNE_DOT_VARIANT);
    const long long pad_small = (long long)((Lx + SB - 1) / SB) * ((Ly + SB - 1) / SB) * SB * SB;
    const long long pad_tiled = (long long)((Lx + TI - 1) / TI) * ((Ly + TJ - 1) / TJ) * TI * TJ;
    // Context path with a reduction length (key positions) that is no multiple of 8 -- sentences come in every
    // length: the per-wavefront kernel's ragged mode reads 4 bytes at a time and needs no alignment; it takes
    // such problems whenever they are short, and all of them when the tiled kernel cannot (length % 4 != 0),
    // where the only alternative is the any-shape kernel (L = 30: 101 us against 22 us).
    const bool ragged_ok = VP && d % 8 != 0 && d <= 80 && (long long)TI * D * max_pitch * 4 < 0xffffffffLL &&
                           (long long)d * D * g.oy.pitch * 4 < 0xffffffffLL;
    const bool small = (small_ok && (pick == 2 || compact_y || (pick != 1 && 100 * pad_small <= 85 * pad_tiled))) ||
                       (ragged_ok && (pick == 2 || compact_y || !fast || (pick != 1 && 100 * pad_small <= 85 * pad_tiled)));
    FAITH_REQUIRE(small || !compact_y, FAITH_ERR_UNSUPPORTED,
                  "%s: a compact value operand needs at most 80 key positions, a head size that is a multiple of 4 and "
                  "16-byte aligned tensors", who);
    if (small) {
        // one 32 x 32 block per wavefront and perturbation coordinate.  Coordinates per wavefront: the
        // count that leaves the busiest CU the least to do -- its share of the workgroups, each costing
        // its coordinates plus about half a coordinate for staging the shared operands (tuner sweeps:
        // this choice is within 5 % of the best count on every shape tried)
        const long long blocks = (long long)B * ((Lx + SB - 1) / SB) * ((Ly + SB - 1) / SB);
        const long long cus = faith::compute_units();
        long long mpw = 1, best = -1;
        for (long long c = 1; c <= 16; ++c) {
            const long long wgs = blocks * ((D + 4 * c - 1) / (4 * c));
            const long long cost = ((wgs + cus - 1) / cus) * (2 * c + 1);
            if (best < 0 || cost < best) { best = cost; mpw = c; }
        }
        const int forced = faith::tune_get(FAITH_TUNE_DOT_COORDS);
        if (forced >= 1 && forced <= 16) mpw = forced;
        const long long grid = blocks * ((D + 4 * mpw - 1) / (4 * mpw));
        FAITH_REQUIRE(grid + b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
        // the constant-term tiles are the trailing workgroups of the same launch while the machine is not
        // filled many times over (one small problem: 30.7 -> 25.1 us); behind a long queue of MFMA workgroups
        // they would only lengthen the tail (batch of 30: 554 -> 567 us), so there they keep their own launch
        const bool fold = blocks * ((D + 3) / 4) <= 16 * cus;      // wavefront-coordinates of work, whatever their grouping
        if (!fold) constant_terms();
        const int dp = (d + 7) / 8 * 8;
        const size_t lds = (size_t)(6 * SB * dp > BT_LDS ? 6 * SB * dp : BT_LDS) * sizeof(float);
        const dim3 gd((unsigned)(grid + (fold ? b_tiles : 0)));
        if constexpr (VP) {
            if (compact_y && d % 8 != 0)
                hipLaunchKernelGGL((dot_w_small<true, true, true>), gd, dim3(256), lds, st, g, (int)mpw, x_sbs ? 1 : 0, (int)grid);
            else if (compact_y)
                hipLaunchKernelGGL((dot_w_small<true, false, true>), gd, dim3(256), lds, st, g, (int)mpw, x_sbs ? 1 : 0, (int)grid);
            else if (d % 8 != 0)
                hipLaunchKernelGGL((dot_w_small<true, true>), gd, dim3(256), lds, st, g, (int)mpw, x_sbs ? 1 : 0, (int)grid);
            else
                hipLaunchKernelGGL((dot_w_small<true, false>), gd, dim3(256), lds, st, g, (int)mpw, x_sbs ? 1 : 0, (int)grid);
        } else {
            hipLaunchKernelGGL((dot_w_small<false, false>), gd, dim3(256), lds, st, g, (int)mpw, x_sbs ? 1 : 0, (int)grid);
        }
    } else if (fast) {
        constant_terms();
        const long long tiles = (long long)B * D * ((Lx + TI - 1) / TI) * ((Ly + TJ - 1) / TJ);
        FAITH_REQUIRE(tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: too many tiles", who);
        const long long resident = 2LL * faith::compute_units();      // 56 KB of LDS each: two per CU
        // the XCD-aware walk deals perturbation coordinates m over the XCDs: needs dim_in % 8 == 0 and
        // a grid that keeps workgroup number % 8 fixed along a walk
        long long grid = tiles < resident ? tiles : resident;
        int xcd_map = 0;
        if (D % 8 == 0 && grid >= 8) {
            grid -= grid % 8;
            xcd_map = 1;
        }
        const bool exact = d % BK == 0 && Lx % TI == 0 && Ly % TJ == 0;
        const long long wx = (long long)B * Lx * D * d, wy = (long long)B * Ly * D * d, wz = (long long)B * Lx * D * Ly;
        // reductions of 32, 64 or 128 with every array under 4 GB: the straight-line kernel (same tiles, same order of
        // summation, same bits); the tuning knob 1 keeps the kernel with run-time extents
        if (exact && xcd_map && pick != 1 && faith::dot_tiled_takes(d) && wx * 4 < 0xffffffffLL && wy * 4 < 0xffffffffLL &&
            wz * 4 < 0xffffffffLL) {
            faith::DotTiledArgs a{};
            a.xlw = x_lw; a.xuw = x_uw; a.ylw = y_lw; a.yuw = y_uw;
            a.x_l = x_l; a.y_l = y_l; a.y_u = y_u;
            a.zlw = z_lw; a.zuw = z_uw;
            const long long nxi = (long long)B * Lx * d, nyi = (long long)B * Ly * d;
            a.x_bytes = (unsigned)(wx * 4); a.y_bytes = (unsigned)(wy * 4); a.z_bytes = (unsigned)(wz * 4);
            a.xi_bytes = (unsigned)(nxi * 4); a.yi_bytes = (unsigned)(nyi * 4);
            a.Lx = Lx; a.Ly = Ly; a.D = D;
            a.xp = g.ox.pitch; a.yp = g.oy.pitch; a.zp = g.oz.pitch;
            // pair t = bb * heads + h of an object with `rows` positions: stacked on the first axis, or heads side by side
            auto strides = [&](const DotArgs::Obj &o, long long rows, long long per_row, unsigned &bs, unsigned &hs) {
                if (o.heads == 1) { hs = (unsigned)(rows * per_row * o.pitch); bs = (unsigned)(hs * (long long)heads); }
                else { bs = (unsigned)(rows * per_row * o.pitch); hs = (unsigned)o.width; }
            };
            strides(g.ox, Lx, D, a.xw_bs, a.xw_hs);  strides(g.ox, Lx, 1, a.xi_bs, a.xi_hs);
            strides(g.oy, y_len, D, a.yw_bs, a.yw_hs);  strides(g.oy, y_len, 1, a.yi_bs, a.yi_hs);
            strides(g.oz, Lx, D, a.zw_bs, a.zw_hs);
            a.heads = heads; a.batches = B / heads;
            a.total_tiles = (int)tiles;
            faith::dot_tiled_launch(VP, d, a, (int)grid, st);
        } else if (exact)
            hipLaunchKernelGGL((dot_w<VP, true>), dim3((unsigned)grid), dim3(NTHREADS), 0, st, g, (int)tiles, xcd_map);
        else
            hipLaunchKernelGGL((dot_w<VP, false>), dim3((unsigned)grid), dim3(NTHREADS), 0, st, g, (int)tiles, xcd_map);
    } else {
        constant_terms();
        const long long blocks = (nw + 255) / 256;
        hipLaunchKernelGGL(dot_w_simple<VP>, dim3((unsigned)(blocks < 65536 ? blocks : 65536)), dim3(256), 0, st, g);
    }
    return faith::check_launch(who);
}

// ------------------------------------------------------------------------------------------
// Transposed layout: what the reference's adapters hand to its kernels (Bounds.py:1279-1290, :1319-1329;
// kernel.cpp:133-241).  Coefficients are [B, L, K, D_in] with the perturbation coordinate m contiguous,
// K the reduction axis (head size for the scores; key positions for the context, where y is the value
// object already transposed to [B, width, keys, D_in]), and the result is z [B, Lx, Ly, D_in]:
//     z[i, j, m] = sum_k  x[i, k, m] a[j, k] + b[i, k] y[j, k, m]        (a, b split by sign as above).
// A fixed-m slice of an operand is a 4-byte gather here, so the MFMA tiling of the natural layout (rows i,
// columns j, one m per tile) would read 4 bytes per 128-byte line.  Lanes run along m instead: every load and
// store of a wavefront is one contiguous 256-byte run, the coefficients a[j, k], b[i, k] are wave-uniform
// (scalar loads), and each lane keeps an RI x RJ block of (i, j) pairs for its m in registers -- 8 RI RJ
// fused multiply-adds per 2 (RI + RJ) loads.  Vector ALU, not MFMA: the kernel for any shape in this layout;
// shapes of whole blocks take the two MFMA launches of dot_transposed.hip (x terms with i fixed, y terms with j
// fixed: each alone is a matrix product whose operands need no re-layout).
// ------------------------------------------------------------------------------------------
struct DotTArgs {
    const float *xlw, *xuw, *ylw, *yuw;   // [B, Lx, K, D], [B, Ly, K, D]
    const float *x_l, *y_l, *y_u;         // [B, Lx, K], [B, Ly, K]
    float *zlw, *zuw;                     // [B, Lx, Ly, D]
    int B, Lx, Ly, K, D;
    int mw;                               // wavefronts of a workgroup along m (1, 2 or 4); the others along j
    int n_i, n_j, n_m;                    // blocks along i, j, m
};

template <int RI, int RJ>
__global__ void __launch_bounds__(256) dot_w_transposed(const DotTArgs g) {
    const int lane = threadIdx.x % 64;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);     // wave-uniform by construction
    const int wm = wave % g.mw, wj = wave / g.mw, jw = 4 / g.mw;
    int blk = blockIdx.x;
    const int mb = blk % g.n_m;  blk /= g.n_m;
    const int jb = blk % g.n_j;  blk /= g.n_j;
    const int ib = blk % g.n_i;
    const int t = blk / g.n_i;
    const int m = (mb * g.mw + wm) * 64 + lane;
    const int i0 = ib * RI, j0 = (jb * jw + wj) * RJ;
    if (j0 >= g.Ly) return;                                  // a wavefront without columns (no barrier below)
    const bool m_ok = m < g.D;
    const int mc = m_ok ? m : g.D - 1;                       // out-of-range lanes read a valid address, store nothing

    // Buffer addressing: one window per tensor and (batch, head) pair, a wave-uniform byte offset per row
    // (scalar registers, advanced by one k per step) and the lane's own offset m.  Rows past the end repeat
    // the last one; their results are not stored.  The coefficients a[j, k], b[i, k] are scalar loads.
    const size_t xh = (size_t)g.Lx * g.K * g.D, yh = (size_t)g.Ly * g.K * g.D;      // floats of one head
    const __amdgpu_buffer_rsrc_t wxl = window(g.xlw + t * xh, clamp32(xh * 4)), wxu = window(g.xuw + t * xh, clamp32(xh * 4));
    const __amdgpu_buffer_rsrc_t wyl = window(g.ylw + t * yh, clamp32(yh * 4)), wyu = window(g.yuw + t * yh, clamp32(yh * 4));
    // the concrete intervals were written by an earlier launch and do not change during this one: read through
    // the constant address space, a wave-uniform address there is a scalar load
    typedef const float __attribute__((address_space(4))) *uniform_ptr;
    const uniform_ptr cb = (uniform_ptr)(g.x_l + (size_t)t * g.Lx * g.K);
    const uniform_ptr cal = (uniform_ptr)(g.y_l + (size_t)t * g.Ly * g.K), cau = (uniform_ptr)(g.y_u + (size_t)t * g.Ly * g.K);
    const unsigned vm = (unsigned)mc * 4u, kstep = (unsigned)g.D * 4u;
    unsigned xo[RI], yo[RJ], bo[RI], ao[RJ];
#pragma unroll
    for (int a = 0; a < RI; ++a) {
        const unsigned i = i0 + a < g.Lx ? i0 + a : g.Lx - 1;
        xo[a] = i * (unsigned)g.K * kstep;
        bo[a] = i * (unsigned)g.K;
    }
#pragma unroll
    for (int c = 0; c < RJ; ++c) {
        const unsigned j = j0 + c < g.Ly ? j0 + c : g.Ly - 1;
        yo[c] = j * (unsigned)g.K * kstep;
        ao[c] = j * (unsigned)g.K;
    }
    float zl[RI][RJ], zu[RI][RJ];
#pragma unroll
    for (int a = 0; a < RI; ++a)
#pragma unroll
        for (int c = 0; c < RJ; ++c) zl[a][c] = zu[a][c] = 0.f;

#pragma unroll 1
    for (int k = 0; k < g.K; ++k) {
        float xl[RI], xu[RI], yl[RJ], yu[RJ], bp[RI], bn[RI], alp[RJ], aln[RJ], aup[RJ], aun[RJ];
#pragma unroll
        for (int a = 0; a < RI; ++a) {
            xl[a] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wxl, vm, xo[a], 0));
            xu[a] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wxu, vm, xo[a], 0));
            const float b = cb[bo[a] + k];
            bp[a] = pos1(b);
            bn[a] = neg1(b);
            xo[a] += kstep;
        }
#pragma unroll
        for (int c = 0; c < RJ; ++c) {
            yl[c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wyl, vm, yo[c], 0));
            yu[c] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(wyu, vm, yo[c], 0));
            const float al = cal[ao[c] + k], au = cau[ao[c] + k];
            alp[c] = pos1(al);  aln[c] = neg1(al);
            aup[c] = pos1(au);  aun[c] = neg1(au);
            yo[c] += kstep;
        }
#pragma unroll
        for (int a = 0; a < RI; ++a)
#pragma unroll
            for (int c = 0; c < RJ; ++c) {
                float l = zl[a][c], u = zu[a][c];
                l = __builtin_fmaf(xl[a], alp[c], l);  u = __builtin_fmaf(xu[a], aup[c], u);
                l = __builtin_fmaf(xu[a], aln[c], l);  u = __builtin_fmaf(xl[a], aun[c], u);
                l = __builtin_fmaf(bp[a], yl[c], l);   u = __builtin_fmaf(bp[a], yu[c], u);
                l = __builtin_fmaf(bn[a], yu[c], l);   u = __builtin_fmaf(bn[a], yl[c], u);
                zl[a][c] = l;  zu[a][c] = u;
            }
    }
    if (!m_ok) return;
#pragma unroll
    for (int a = 0; a < RI; ++a) {
        if (i0 + a >= g.Lx) break;
#pragma unroll
        for (int c = 0; c < RJ; ++c) {
            if (j0 + c >= g.Ly) break;
            const size_t z = (((size_t)t * g.Lx + i0 + a) * g.Ly + j0 + c) * g.D + m;
            __builtin_nontemporal_store(zl[a][c], g.zlw + z);
            __builtin_nontemporal_store(zu[a][c], g.zuw + z);
        }
    }
}

// Both entry points in the transposed layout: `K` is the reduction length (head size for the scores, key
// positions for the context), `Ly` the number of result columns (key positions / width of the values).
int dot_entry_transposed(const char *who, float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                         const float *x_ub, const float *y_lb, const float *y_ub, const float *x_lw, const float *x_uw,
                         const float *y_lw, const float *y_uw, float *z_lb, float *z_ub, float *z_lw, float *z_uw, int B,
                         int Lx, int Ly, int K, int D, float epsilon, int q, int words, void *stream) {
    FAITH_NOT_NULL(x_l); FAITH_NOT_NULL(y_l); FAITH_NOT_NULL(y_u);      // x_u may be NULL: not wanted
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub);
    FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_NOT_NULL(z_lb); FAITH_NOT_NULL(z_ub); FAITH_NOT_NULL(z_lw); FAITH_NOT_NULL(z_uw);
    FAITH_ALIGNED4(x_lw); FAITH_ALIGNED4(x_uw); FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_ALIGNED4(z_lw); FAITH_ALIGNED4(z_uw); FAITH_ALIGNED4(z_lb); FAITH_ALIGNED4(z_ub);
    FAITH_REQUIRE(B > 0 && Lx > 0 && Ly > 0 && K > 0 && D > 0, FAITH_ERR_SHAPE,
                  "%s: batch=%d rows of x=%d columns of z=%d reduction length=%d dim_in=%d must be positive", who, B, Lx,
                  Ly, K, D);
    FAITH_REQUIRE((long long)B * (Lx > Ly ? Lx : Ly) * K <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "%s: batch * length * reduction length exceeds 2^31", who);
    FAITH_REQUIRE(words >= 1 && (D == 1 || D % words == 0), FAITH_ERR_SHAPE, "%s: words=%d must divide dim_in=%d", who, words, D);
    // every requirement is checked before the first launch: a call that is refused has written nothing
    const long long b_tiles = (long long)B * ((Lx + BT_T - 1) / BT_T) * ((Ly + BT_T - 1) / BT_T);
    FAITH_REQUIRE(b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
    FAITH_REQUIRE(D == 1 || (long long)(Lx > Ly ? Lx : Ly) * K * D * 4 < 0xffffffffLL, FAITH_ERR_UNSUPPORTED,
                  "%s: the coefficients of one batch element exceed 4 GB in the transposed layout (32-bit offsets)", who);
    constexpr int RI = 4, RJ = 8;
    DotTArgs a{x_lw, x_uw, y_lw, y_uw, x_l, y_l, y_u, z_lw, z_uw, B, Lx, Ly, K, D};
    a.mw = D > 128 ? 4 : D > 64 ? 2 : 1;
    a.n_i = (Lx + RI - 1) / RI;
    a.n_j = (Ly + RJ * (4 / a.mw) - 1) / (RJ * (4 / a.mw));
    a.n_m = (D + 64 * a.mw - 1) / (64 * a.mw);
    const long long grid = (long long)B * a.n_i * a.n_j * a.n_m;
    FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
    hipStream_t st = static_cast<hipStream_t>(stream);

    // concrete intervals of both objects: [B * L, K] neurons whose D_in coefficients are contiguous
    const bool empty_blocks = D == 1 && words > 1;      // Bounds.py:319-326 with dim_in // words == 0: the constant terms
    const float eps = empty_blocks ? 0.f : epsilon;
    const int w = empty_blocks ? 1 : words;
    int rc = faith::concretize_pair(x_lb, x_ub, x_lw, x_uw, x_l, x_u, B * Lx, nullptr, nullptr, nullptr, nullptr, nullptr,
                                    nullptr, 0, D, K, 0, eps, q, w, stream, FAITH_LAYOUT_TRANSPOSED);
    if (rc != FAITH_OK) return rc;
    rc = faith_concretize(y_lb, y_ub, y_lw, y_uw, y_l, y_u, B * Ly, D, K, eps, q, w, FAITH_LAYOUT_TRANSPOSED, stream);
    if (rc != FAITH_OK) return rc;

    // constant terms and the dim_in == 1 shortcut do not involve the coefficient layout: the kernels of the
    // natural layout serve (scores form: rows of x and of y, reduction over their last axis)
    DotArgs g{x_lw, x_uw, y_lw, y_uw, x_lb, x_ub, y_lb, y_ub, x_l, y_l, y_u, z_lw, z_uw, z_lb, z_ub, B, Lx, Ly, D, K};
    g.ox = {K, 1, K};
    g.oy = {K, 1, K};
    g.oz = {Ly, 1, Ly};
    g.heads = 1;
    g.side_by_side = 0;
    if (D == 1) {
        const long long n = (long long)B * Lx * Ly;      // z_lw [B, Lx, Ly, 1] and [B, Lx, 1, Ly] coincide
        hipLaunchKernelGGL(dot_interval<false>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, g);
        return faith::check_launch(who);
    }
    hipLaunchKernelGGL(dot_b<false>, dim3((unsigned)b_tiles), dim3(256), 0, st, g);
    // whole blocks everywhere: the MFMA kernels (knob value 3 keeps the vector-ALU kernel)
    if (faith::tune_get(FAITH_TUNE_DOT_VARIANT) != 3 && faith::dot_transposed_mfma_takes(Lx, Ly, K, D)) {
        const faith::DotTransposedArgs ta{x_lw, x_uw, y_lw, y_uw, x_l, y_l, y_u, z_lw, z_uw, B, Lx, Ly, K, D};
        if (faith::dot_transposed_mfma_launch(ta, st)) return faith::check_launch(who);
    }
    hipLaunchKernelGGL((dot_w_transposed<RI, RJ>), dim3((unsigned)grid), dim3(256), 0, st, a);
    return faith::check_launch(who);
}


// ---------------------------------------------------------------------------------------------------------
// Scores of a query and a key whose coefficients vanish outside P positions of every batch element: the
// input of a verification query has coefficients at the perturbed position(s) only (VerifierForward.py:127-156),
// and layer norm and dense layers keep it that way.  In Bounds.py:761-818 the x terms of z[i, m, j] are sums over
// x.lw[i, m, :] and the y terms over y.lw[j, m, :], so z_lw[i, :, j] is zero unless i or j is one of those positions:
//     i in S:  z[i, m, j] += sum_k a(j, k) split by sign against x.lw / x.uw [i, m, k]     (every j)
//     j in S:  z[i, m, j] += sum_k b(i, k) split by sign against y.lw / y.uw [j, m, k]     (every i)
// Only the rows of S exist in memory ([batch, P, D, heads * size], heads side by side).  A workgroup writes the
// coordinates m0 ... m0 + 127 of one (batch element, head, i): first the P column values per coordinate (four lanes
// per dot product), then the [128 x L] block, 16 bytes per lane -- zeros, the column values where j is in S and, in the
// HEAVY launch (one workgroup per row i in S), the full row of x terms against a(j, k) staged in LDS as [k][j].
// The LIGHT launch covers every i and leaves the rows of S to the other.  The work is 1 / L of the dense
// contraction: this is a vector-ALU kernel bound by writing z.
struct CompactArgs {
    const float *xlw, *xuw, *ylw, *yuw;    // [batch, P, D, heads * size]
    const float *x_l, *y_l, *y_u;          // [batch, L, heads * size]
    const long long *positions;            // [batch, P], distinct within a batch element; outside 0 ... L-1: no such row
    float *zlw, *zuw;                      // [batch * heads, L, D, L]
    int L, P, D, heads, size, chunks;
};
constexpr int CS_MC = 128;

template <bool HEAVY>
__global__ void __launch_bounds__(256) scores_compact(const CompactArgs g) {
    extern __shared__ __align__(16) float cs[];
    const int L = g.L, P = g.P, size = g.size, pitch = g.heads * g.size;
    float *col_l = cs, *col_u = cs + P * CS_MC;                       // [P][CS_MC]
    float *alp = cs + 2 * P * CS_MC, *aln = alp + size * L, *aup = aln + size * L, *aun = aup + size * L;   // [size][L] each
    int pid = blockIdx.x;
    const int c = pid % g.chunks;  pid /= g.chunks;
    const int r = pid % (HEAVY ? P : L);  pid /= (HEAVY ? P : L);
    const int t = pid, b = t / g.heads, h = t - b * g.heads;
    const long long *pos = g.positions + (size_t)b * P;
    int i = r, pi = -1;
    if (HEAVY) {
        const long long at = pos[r];
        if (at < 0 || at >= L) return;                                // no such row (uniform over the workgroup)
        i = (int)at;  pi = r;
    } else {
        for (int p = 0; p < P; ++p)
            if (pos[p] == i) return;                                  // a row of S: the other launch writes it
    }
    const int m0 = c * CS_MC, tid = threadIdx.x;

    // ---- column values: b(i, :) against the key's rows of S
    const float *beta = g.x_l + ((size_t)b * L + i) * pitch + (size_t)h * size;
    for (int e = tid; e < 4 * P * CS_MC; e += 256) {                  // 4 * CS_MC is a multiple of 256: no lane sits out
        const int part = e % 4, ml = (e / 4) % CS_MC, p = e / (4 * CS_MC);
        float sl = 0.f, su = 0.f;
        if (m0 + ml < g.D) {
            const size_t row = (((size_t)b * P + p) * g.D + m0 + ml) * pitch + (size_t)h * size;
            for (int k = 4 * part; k < size; k += 16) {
                const float4 bt = *reinterpret_cast<const float4 *>(beta + k);
                const float4 yl = *reinterpret_cast<const float4 *>(g.ylw + row + k);
                const float4 yu = *reinterpret_cast<const float4 *>(g.yuw + row + k);
#define FAITH_TERM(F)                                                        \
    {                                                                        \
        const float bp = fmaxf(bt.F, 0.f), bn = fminf(bt.F, 0.f);            \
        sl += bp * yl.F + bn * yu.F;                                         \
        su += bp * yu.F + bn * yl.F;                                         \
    }
                FAITH_TERM(x) FAITH_TERM(y) FAITH_TERM(z) FAITH_TERM(w)
#undef FAITH_TERM
            }
        }
        sl += __shfl_xor(sl, 1);  su += __shfl_xor(su, 1);
        sl += __shfl_xor(sl, 2);  su += __shfl_xor(su, 2);
        if (part == 0) { col_l[p * CS_MC + ml] = sl;  col_u[p * CS_MC + ml] = su; }
    }
    if (HEAVY) {
        // a_l, a_u of this head, split by sign, as [k][j]
        for (int e = tid; e < size * L; e += 256) {
            const int j = e / size, k = e % size;
            const size_t o = ((size_t)b * L + j) * pitch + (size_t)h * size + k;
            const float al = g.y_l[o], au = g.y_u[o];
            alp[k * L + j] = fmaxf(al, 0.f);  aln[k * L + j] = fminf(al, 0.f);
            aup[k * L + j] = fmaxf(au, 0.f);  aun[k * L + j] = fminf(au, 0.f);
        }
    }
    __syncthreads();

    // ---- the block of z: 16 bytes (four columns j of one coordinate m) per lane and step
    const size_t z0 = (((size_t)t * L + i) * g.D + m0) * L;
    const int rows = min(CS_MC, g.D - m0);
    for (int e4 = tid; e4 < rows * L / 4; e4 += 256) {
        const int ml = (e4 * 4) / L, j0 = (e4 * 4) % L;
        float vl[4] = {0.f, 0.f, 0.f, 0.f}, vu[4] = {0.f, 0.f, 0.f, 0.f};
        if (HEAVY) {
            const size_t row = (((size_t)b * P + pi) * g.D + m0 + ml) * pitch + (size_t)h * size;
            for (int k = 0; k < size; k += 4) {
                const float4 xl4 = *reinterpret_cast<const float4 *>(g.xlw + row + k);
                const float4 xu4 = *reinterpret_cast<const float4 *>(g.xuw + row + k);
                const float xl[4] = {xl4.x, xl4.y, xl4.z, xl4.w}, xu[4] = {xu4.x, xu4.y, xu4.z, xu4.w};
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    const int o = (k + kk) * L + j0;
                    const float4 a1 = *reinterpret_cast<const float4 *>(alp + o), a2 = *reinterpret_cast<const float4 *>(aln + o);
                    const float4 a3 = *reinterpret_cast<const float4 *>(aup + o), a4 = *reinterpret_cast<const float4 *>(aun + o);
                    vl[0] += a1.x * xl[kk] + a2.x * xu[kk];  vu[0] += a3.x * xu[kk] + a4.x * xl[kk];
                    vl[1] += a1.y * xl[kk] + a2.y * xu[kk];  vu[1] += a3.y * xu[kk] + a4.y * xl[kk];
                    vl[2] += a1.z * xl[kk] + a2.z * xu[kk];  vu[2] += a3.z * xu[kk] + a4.z * xl[kk];
                    vl[3] += a1.w * xl[kk] + a2.w * xu[kk];  vu[3] += a3.w * xu[kk] + a4.w * xl[kk];
                }
            }
        }
        for (int p = 0; p < P; ++p) {
            const long long jp = pos[p] - j0;
            if (jp >= 0 && jp < 4) {
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (q == (int)jp) { vl[q] += col_l[p * CS_MC + ml];  vu[q] += col_u[p * CS_MC + ml]; }
            }
        }
        *reinterpret_cast<float4 *>(g.zlw + z0 + (size_t)e4 * 4) = make_float4(vl[0], vl[1], vl[2], vl[3]);
        *reinterpret_cast<float4 *>(g.zuw + z0 + (size_t)e4 * 4) = make_float4(vu[0], vu[1], vu[2], vu[3]);
    }
}

// The HEAVY launch on the matrix unit (L and D multiples of 32, head size 32 or 64): for a row i in S the x terms
// are a matrix product with rows m -- [D x size] coefficient rows of x against the [size x L] intervals of the key,
// split by sign --, so a wavefront takes 32 coordinates m and, in turn, every block of 32 columns j: its x fragments
// and the key's intervals come straight from global memory in MFMA layout (lane (row, half) holds k = 8 s + 4 half
// .. + 3 of its row), four products per K-pair as in dot_w_small.  The vector-ALU version above walks the reduction
// with a global load per four k in every lane's chain (32 us for one query's four heads); this one has its loads
// in flight together and 128 MFMAs per block.  A workgroup is four such wavefronts (128 coordinates) and first
// forms the column values of its coordinates (the y terms) as the other launch does.
template <int NS>                                                     // NS = head size / 8: K-steps
__global__ void __launch_bounds__(256) scores_compact_heavy_mfma(const CompactArgs g) {
    extern __shared__ __align__(16) float cs[];
    constexpr int size = 8 * NS;
    const int L = g.L, P = g.P, pitch = g.heads * size;
    float *col_l = cs, *col_u = cs + P * CS_MC;                       // [P][CS_MC]
    int pid = blockIdx.x;
    const int c = pid % g.chunks;  pid /= g.chunks;
    const int pi = pid % P;  pid /= P;
    const int t = pid, b = t / g.heads, h = t - b * g.heads;
    const long long *pos = g.positions + (size_t)b * P;
    const long long at = pos[pi];
    if (at < 0 || at >= L) return;                                    // no such row (uniform over the workgroup)
    const int i = (int)at;
    const int m0 = c * CS_MC, tid = threadIdx.x;
    const int lane = tid % 64, wv = tid / 64;
    const int fi = lane % 32, fh = lane / 32;
    const int mb = m0 + 32 * wv;                                      // this wavefront's 32 coordinates
    const bool active = mb < g.D;

    // ---- the wavefront's x fragments (they serve every block of columns) and the key's intervals of the first block:
    // asked for before anything else, so that they arrive under the column values
    const size_t xrow = (((size_t)b * P + pi) * g.D + (active ? mb + fi : 0)) * pitch + (size_t)h * size + 4 * fh;
    float4 xl[NS], xu[NS], al[NS], au[NS];
    auto fetch_a = [&](int j0) __attribute__((always_inline)) {
        const size_t arow = ((size_t)b * L + j0 + fi) * pitch + (size_t)h * size + 4 * fh;
#pragma unroll
        for (int s_ = 0; s_ < NS; ++s_) {
            al[s_] = *reinterpret_cast<const float4 *>(g.y_l + arow + 8 * s_);
            au[s_] = *reinterpret_cast<const float4 *>(g.y_u + arow + 8 * s_);
        }
    };
    if (active) {
#pragma unroll
        for (int s_ = 0; s_ < NS; ++s_) {
            xl[s_] = *reinterpret_cast<const float4 *>(g.xlw + xrow + 8 * s_);
            xu[s_] = *reinterpret_cast<const float4 *>(g.xuw + xrow + 8 * s_);
        }
        fetch_a(0);
    }

    // ---- column values: b(i, :) against the key's rows of S; the loads of a dot product's quarter go out together
    const float *beta = g.x_l + ((size_t)b * L + i) * pitch + (size_t)h * size;
    for (int e = tid; e < 4 * P * CS_MC; e += 256) {
        const int part = e % 4, ml = (e / 4) % CS_MC, p = e / (4 * CS_MC);
        float sl = 0.f, su = 0.f;
        if (m0 + ml < g.D) {
            const size_t row = (((size_t)b * P + p) * g.D + m0 + ml) * pitch + (size_t)h * size;
            constexpr int NQ = (size + 15) / 16;
            float4 bt[NQ], yl[NQ], yu[NQ];
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const int k = 4 * part + 16 * q;
                const bool in = k < size;
                const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
                bt[q] = in ? *reinterpret_cast<const float4 *>(beta + k) : zero;
                yl[q] = in ? *reinterpret_cast<const float4 *>(g.ylw + row + k) : zero;
                yu[q] = in ? *reinterpret_cast<const float4 *>(g.yuw + row + k) : zero;
            }
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
#define FAITH_TERM(F)                                                        \
    {                                                                        \
        const float bp = fmaxf(bt[q].F, 0.f), bn = fminf(bt[q].F, 0.f);      \
        sl += bp * yl[q].F + bn * yu[q].F;                                   \
        su += bp * yu[q].F + bn * yl[q].F;                                   \
    }
                FAITH_TERM(x) FAITH_TERM(y) FAITH_TERM(z) FAITH_TERM(w)
#undef FAITH_TERM
            }
        }
        sl += __shfl_xor(sl, 1);  su += __shfl_xor(su, 1);
        sl += __shfl_xor(sl, 2);  su += __shfl_xor(su, 2);
        if (part == 0) { col_l[p * CS_MC + ml] = sl;  col_u[p * CS_MC + ml] = su; }
    }
    __syncthreads();
    if (!active) return;

    for (int j0 = 0; j0 < L; j0 += 32) {
        floatx16 cl, cu;
#pragma unroll
        for (int r = 0; r < 16; ++r) cl[r] = cu[r] = 0.f;
#pragma unroll
        for (int s_ = 0; s_ < NS; ++s_) {
#define FAITH_STEP(F)                                                 \
    cl = mfma(xl[s_].F, fmaxf(al[s_].F, 0.f), cl);                    \
    cu = mfma(xu[s_].F, fmaxf(au[s_].F, 0.f), cu);                    \
    cl = mfma(xu[s_].F, fminf(al[s_].F, 0.f), cl);                    \
    cu = mfma(xl[s_].F, fminf(au[s_].F, 0.f), cu);
            FAITH_STEP(x) FAITH_STEP(y) FAITH_STEP(z) FAITH_STEP(w)
#undef FAITH_STEP
        }
        const int jcol = j0 + fi;
        if (j0 + 32 < L) fetch_a(j0 + 32);                            // the next block's intervals under this block's stores
        // register r is coordinate 8 (r / 4) + 4 fh + r % 4 of the block, lanes run along j; the column of a key
        // position of S takes its column value on top
        for (int p = 0; p < P; ++p) {
            if (pos[p] == (long long)jcol) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int ml = 32 * wv + 8 * (r / 4) + 4 * fh + (r % 4);
                    cl[r] += col_l[p * CS_MC + ml];
                    cu[r] += col_u[p * CS_MC + ml];
                }
            }
        }
        const size_t z0 = (((size_t)t * L + i) * g.D + mb) * L + jcol;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const size_t o = z0 + (size_t)(8 * (r / 4) + 4 * fh + (r % 4)) * L;
            g.zlw[o] = cl[r];
            g.zuw[o] = cu[r];
        }
    }
}

}  // namespace

extern "C" int faith_dot_product_verification_QK(float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                                                 const float *x_ub, const float *y_lb, const float *y_ub,
                                                 const float *x_lw, const float *x_uw, const float *y_lw,
                                                 const float *y_uw, float *z_lb, float *z_ub, float *z_lw,
                                                 float *z_uw, int batch_size, int length_x, int length_y,
                                                 int dim_out, int dim_in, float epsilon, int q, int words,
                                                 int layout, void *stream) {
    if (layout == FAITH_LAYOUT_TRANSPOSED)
        return dot_entry_transposed("faith_dot_product_verification_QK", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw,
                                    x_uw, y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size, length_x, length_y, dim_out,
                                    dim_in, epsilon, q, words, stream);
    FAITH_REQUIRE(layout == FAITH_LAYOUT_NATURAL, FAITH_ERR_UNSUPPORTED, "faith_dot_product_verification_QK: unknown layout %d", layout);
    return dot_entry<false>("faith_dot_product_verification_QK", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw,
                            y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size, length_x, length_y, dim_out, dim_in, epsilon,
                            q, words, 0, 1, stream);
}

extern "C" int faith_dot_product_verification_V(float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                                                const float *x_ub, const float *y_lb, const float *y_ub,
                                                const float *x_lw, const float *x_uw, const float *y_lw,
                                                const float *y_uw, float *z_lb, float *z_ub, float *z_lw,
                                                float *z_uw, int batch_size, int length_x, int length_k, int dim_out,
                                                int dim_in, float epsilon, int q, int words, int layout, void *stream) {
    if (layout == FAITH_LAYOUT_TRANSPOSED)      // y is the value object transposed: [batch, dim_out, length_k, dim_in]
        return dot_entry_transposed("faith_dot_product_verification_V", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw,
                                    x_uw, y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size, length_x, dim_out, length_k,
                                    dim_in, epsilon, q, words, stream);
    FAITH_REQUIRE(layout == FAITH_LAYOUT_NATURAL, FAITH_ERR_UNSUPPORTED, "faith_dot_product_verification_V: unknown layout %d", layout);
    return dot_entry<true>("faith_dot_product_verification_V", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw,
                           y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size, length_x, dim_out, length_k, dim_in, epsilon,
                           q, words, 0, 1, stream);
}

// ------------------------------------------------------------------------------------------
// An entry point that allocates nothing and takes no scratch from its caller.
//
// faith_dot_product_verification_QK needs four scratch arrays from its caller (the concrete intervals
// x_l, x_u, y_l, y_u).  The variant below keeps them in a file-scope device array instead, for callers
// that cannot allocate: code under HIP graph capture, tight serving loops.  Each GPU holds its own copy
// of the array (4 MiB) at its own address until the process ends; the address is looked up once per
// device, with that device current, and only that address -- never the array's name, which is a
// host-side stand-in -- is handed to kernels.  Nothing in it has to start at zero: every call overwrites
// the part it reads.  Calls that overlap on one GPU share the array and race.
// ------------------------------------------------------------------------------------------
constexpr size_t STATIC_SCRATCH_FLOATS = (size_t)1 << 20;
static __device__ __align__(256) float scratch[STATIC_SCRATCH_FLOATS];

constexpr int MAX_DEVICES = 64;
static float *scratch_ptr[MAX_DEVICES];
static std::mutex scratch_mutex;

// Device address of this GPU's copy of `scratch` (looked up on the first call per device).
static int scratch_address(const char *who, float **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    FAITH_REQUIRE(e == hipSuccess && dev >= 0 && dev < MAX_DEVICES, FAITH_ERR_LAUNCH, "%s: hipGetDevice: %s (device %d)", who,
                  hipGetErrorString(e), dev);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {
        float *p = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
        FAITH_REQUIRE(e == hipSuccess && p != nullptr, FAITH_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch): %s", who,
                      hipGetErrorString(e));
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return FAITH_OK;
}

extern "C" long long faith_static_scratch_bytes(void) { return (long long)(STATIC_SCRATCH_FLOATS * sizeof(float)); }

extern "C" int faith_dot_product_verification_QK_static(const float *x_lb, const float *x_ub, const float *y_lb,
                                                        const float *y_ub, const float *x_lw, const float *x_uw,
                                                        const float *y_lw, const float *y_uw, float *z_lb, float *z_ub,
                                                        float *z_lw, float *z_uw, int batch_size, int length_x,
                                                        int length_y, int dim_out, int dim_in, float epsilon, int q,
                                                        int words, int layout, void *stream) {
    const char *who = "faith_dot_product_verification_QK_static";
    FAITH_REQUIRE(batch_size > 0 && length_x > 0 && length_y > 0 && dim_out > 0 && dim_in > 0, FAITH_ERR_SHAPE,
                  "%s: batch=%d length_x=%d length_y=%d dim_out=%d dim_in=%d must be positive", who, batch_size, length_x,
                  length_y, dim_out, dim_in);
    // three segments (x_l, y_l, y_u: the upper interval of x is not asked for), each rounded up to 64 floats so
    // that every one starts 256-byte aligned
    auto seg = [](long long n) { return (n + 63) / 64 * 64; };
    const long long nx = seg((long long)batch_size * length_x * dim_out), ny = seg((long long)batch_size * length_y * dim_out);
    FAITH_REQUIRE(nx + 2 * ny <= (long long)STATIC_SCRATCH_FLOATS, FAITH_ERR_UNSUPPORTED,
                  "%s: the concrete intervals need %lld floats of scratch (batch * (length_x + 2 * length_y) * dim_out, "
                  "segments rounded to 64), the static array holds %lld; use faith_dot_product_verification_QK with "
                  "caller-owned scratch for this size", who, nx + 2 * ny, (long long)STATIC_SCRATCH_FLOATS);
    float *base = nullptr;
    const int rc = scratch_address(who, &base);
    if (rc != FAITH_OK) return rc;
    float *x_l = base, *x_u = nullptr, *y_l = base + nx, *y_u = base + nx + ny;
    if (layout == FAITH_LAYOUT_TRANSPOSED)
        return dot_entry_transposed(who, x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw, z_lb, z_ub, z_lw,
                                    z_uw, batch_size, length_x, length_y, dim_out, dim_in, epsilon, q, words, stream);
    FAITH_REQUIRE(layout == FAITH_LAYOUT_NATURAL, FAITH_ERR_UNSUPPORTED, "%s: unknown layout %d", who, layout);
    return dot_entry<false>(who, x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw, z_lb, z_ub, z_lw, z_uw,
                            batch_size, length_x, length_y, dim_out, dim_in, epsilon, q, words, 0, 1, stream);
}

extern "C" int faith_attention_scores(float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                                      const float *x_ub, const float *y_lb, const float *y_ub, const float *x_lw,
                                      const float *x_uw, const float *y_lw, const float *y_uw, float *z_lb, float *z_ub,
                                      float *z_lw, float *z_uw, int batch_size, int heads, int length_x, int length_y,
                                      int head_size, int dim_in, float epsilon, int q, int words, void *stream) {
    FAITH_REQUIRE(batch_size > 0 && heads > 0 && (long long)batch_size * heads <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "faith_attention_scores: batch=%d heads=%d out of range", batch_size, heads);
    return dot_entry<false>("faith_attention_scores", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw,
                            z_lb, z_ub, z_lw, z_uw, batch_size * heads, length_x, length_y, head_size, dim_in, epsilon, q,
                            words, HEADS_X | HEADS_Y, heads, stream);
}

extern "C" int faith_attention_context_compact(float *x_l, float *x_u, const float *y_l, const float *y_u,
                                               const float *x_lb, const float *x_ub, const float *y_lb,
                                               const float *y_ub, const float *x_lw, const float *x_uw,
                                               const float *y_lw, const float *y_uw, const long long *positions,
                                               float *z_lb, float *z_ub, float *z_lw, float *z_uw, int batch_size,
                                               int heads, int length_x, int length_k, int n_positions, int head_size,
                                               int dim_in, float epsilon, int q, int words, void *stream) {
    FAITH_REQUIRE(batch_size > 0 && heads > 0 && (long long)batch_size * heads <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "faith_attention_context_compact: batch=%d heads=%d out of range", batch_size, heads);
    FAITH_NOT_NULL(positions);
    return dot_entry<true>("faith_attention_context_compact", x_l, const_cast<float *>(y_l), x_u, const_cast<float *>(y_u),
                           x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw, z_lb, z_ub, z_lw, z_uw, batch_size * heads,
                           length_x, head_size, length_k, dim_in, epsilon, q, words, HEADS_Y | HEADS_Z, heads, stream,
                           positions, n_positions);
}

extern "C" int faith_attention_scores_compact(const float *x_l, const float *y_l, const float *y_u, const float *x_lb,
                                              const float *x_ub, const float *y_lb, const float *y_ub, const float *x_lw,
                                              const float *x_uw, const float *y_lw, const float *y_uw,
                                              const long long *positions, float *z_lb, float *z_ub, float *z_lw,
                                              float *z_uw, int batch_size, int heads, int length, int n_positions,
                                              int head_size, int dim_in, void *stream) {
    const char *who = "faith_attention_scores_compact";
    FAITH_NOT_NULL(x_l); FAITH_NOT_NULL(y_l); FAITH_NOT_NULL(y_u);
    FAITH_NOT_NULL(x_lb); FAITH_NOT_NULL(x_ub); FAITH_NOT_NULL(y_lb); FAITH_NOT_NULL(y_ub);
    FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw); FAITH_NOT_NULL(positions);
    FAITH_NOT_NULL(z_lb); FAITH_NOT_NULL(z_ub); FAITH_NOT_NULL(z_lw); FAITH_NOT_NULL(z_uw);
    FAITH_ALIGNED4(x_lb); FAITH_ALIGNED4(x_ub); FAITH_ALIGNED4(y_lb); FAITH_ALIGNED4(y_ub); FAITH_ALIGNED4(z_lb); FAITH_ALIGNED4(z_ub);
    FAITH_REQUIRE(batch_size > 0 && heads > 0 && length > 0 && n_positions > 0 && head_size > 0 && dim_in > 0, FAITH_ERR_SHAPE,
                  "%s: batch=%d heads=%d length=%d positions=%d head size=%d dim_in=%d must be positive", who, batch_size,
                  heads, length, n_positions, head_size, dim_in);
    const long long B = (long long)batch_size * heads;
    FAITH_REQUIRE(B <= 0x7fffffffLL && B * length * dim_in <= 0x7fffffffLL && (long long)heads * head_size <= 0x7fffffffLL &&
                  (long long)batch_size * n_positions * dim_in <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "%s: batch*heads*length*dim_in exceeds 2^31", who);
    // the kernel reads and writes 16 bytes at a time and keeps the key's intervals of one head in LDS; dim_in == 1 is the
    // interval shortcut of the dense entry point (Bounds.py:711-721), which this one does not have
    const size_t lds = ((size_t)2 * n_positions * CS_MC + (size_t)4 * head_size * length) * sizeof(float);
    FAITH_REQUIRE(dim_in > 1 && length % 4 == 0 && head_size % 4 == 0 && lds <= 160 * 1024 && ((uintptr_t)positions & 7) == 0 &&
                  faith::aligned(x_l, 16) && faith::aligned(y_l, 16) && faith::aligned(y_u, 16) &&
                  faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) && faith::aligned(y_lw, 16) &&
                  faith::aligned(y_uw, 16) && faith::aligned(z_lw, 16) && faith::aligned(z_uw, 16), FAITH_ERR_UNSUPPORTED,
                  "%s: needs dim_in > 1, length and head size multiples of 4, 16-byte aligned tensors and "
                  "8 * positions * 128 + 16 * head size * length <= 163840 bytes of LDS", who);
    FAITH_REQUIRE(faith::reserve_lds(scores_compact<true>, lds), FAITH_ERR_UNSUPPORTED,
                  "%s: %zu bytes of LDS per workgroup could not be reserved", who, lds);
    hipStream_t st = static_cast<hipStream_t>(stream);
    CompactArgs c{x_lw, x_uw, y_lw, y_uw, x_l, y_l, y_u, positions, z_lw, z_uw, length, n_positions, dim_in, heads, head_size,
                  (dim_in + CS_MC - 1) / CS_MC};
    const long long light = B * length * c.chunks, heavy = B * n_positions * c.chunks;
    FAITH_REQUIRE(light <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
    const long long b_tiles = B * ((length + BT_T - 1) / BT_T) * ((length + BT_T - 1) / BT_T);
    FAITH_REQUIRE(b_tiles <= 0x7fffffffLL, FAITH_ERR_SHAPE, "%s: grid too large", who);
    // rows of S: on the matrix unit where the blocks are whole (knob value 4 keeps the vector-ALU kernel)
    const bool on_mfma = length % 32 == 0 && dim_in % 32 == 0 && (head_size == 32 || head_size == 64) &&
                         faith::tune_get(FAITH_TUNE_DOT_VARIANT) != 4;
    const size_t col_lds = (size_t)2 * n_positions * CS_MC * sizeof(float);
    if (on_mfma && head_size == 64)
        hipLaunchKernelGGL(scores_compact_heavy_mfma<8>, dim3((unsigned)heavy), dim3(256), col_lds, st, c);
    else if (on_mfma)
        hipLaunchKernelGGL(scores_compact_heavy_mfma<4>, dim3((unsigned)heavy), dim3(256), col_lds, st, c);
    else
        hipLaunchKernelGGL(scores_compact<true>, dim3((unsigned)heavy), dim3(256), lds, st, c);
    hipLaunchKernelGGL(scores_compact<false>, dim3((unsigned)light), dim3(256), (size_t)2 * n_positions * CS_MC * sizeof(float), st, c);
    // constant terms: the dense kernel (it reads constants and intervals only)
    DotArgs g{nullptr, nullptr, nullptr, nullptr, x_lb, x_ub, y_lb, y_ub, x_l, y_l, y_u, nullptr, nullptr, z_lb, z_ub,
              (int)B, length, length, dim_in, head_size};
    g.ox = {heads * head_size, heads, head_size};
    g.oy = {heads * head_size, heads, head_size};
    g.oz = {length, 1, length};
    g.heads = heads;
    g.side_by_side = HEADS_X | HEADS_Y;
    hipLaunchKernelGGL(dot_b<false>, dim3((unsigned)b_tiles), dim3(256), 0, st, g);
    return faith::check_launch(who);
}

extern "C" int faith_attention_context(float *x_l, float *y_l, float *x_u, float *y_u, const float *x_lb,
                                       const float *x_ub, const float *y_lb, const float *y_ub, const float *x_lw,
                                       const float *x_uw, const float *y_lw, const float *y_uw, float *z_lb, float *z_ub,
                                       float *z_lw, float *z_uw, int batch_size, int heads, int length_x, int length_k,
                                       int head_size, int dim_in, float epsilon, int q, int words, void *stream) {
    FAITH_REQUIRE(batch_size > 0 && heads > 0 && (long long)batch_size * heads <= 0x7fffffffLL, FAITH_ERR_SHAPE,
                  "faith_attention_context: batch=%d heads=%d out of range", batch_size, heads);
    return dot_entry<true>("faith_attention_context", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw,
                           z_lb, z_ub, z_lw, z_uw, batch_size * heads, length_x, head_size, length_k, dim_in, epsilon, q,
                           words, HEADS_Y | HEADS_Z, heads, stream);
}

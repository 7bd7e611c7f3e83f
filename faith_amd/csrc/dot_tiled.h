// The straight-line tiled kernel of the dot-product bounds (dot_tiled.hip) as dot.hip sees it.
#pragma once
#include "common.h"

namespace faith {

// Operands of one launch.  Every array is addressed through one buffer descriptor over the whole array and
// 32-bit byte offsets from its first element, so each array must span less than 4 GB (the entry point checks).
struct DotTiledArgs {
    const float *xlw, *xuw, *ylw, *yuw;             // coefficients
    const float *x_l, *y_l, *y_u;                   // concrete intervals: b = x_l, a_l = y_l, a_u = y_u
    // planes, split by sign once per call (nullptr: split by the staging threads, once per tile and K-step):
    // |b| in the layout of x_l; max(a_l, 0), min(a_l, 0), max(a_u, 0), min(a_u, 0) in the layout of y_l
    const float *b_abs, *al_pos, *al_neg, *au_pos, *au_neg;
    float *zlw, *zuw;
    unsigned x_bytes, y_bytes, xi_bytes, yi_bytes, z_bytes;      // sizes of the arrays: coefficients, intervals, result
    int Lx, Ly, D;                                  // rows of x, columns of z, dim_in; the reduction length is 8 * NK
    int xp, yp, zp;                                 // floats from one row to the next
    // first element of (batch element bb, head h) in floats: bb * batch stride + h * head stride
    unsigned xw_bs, xw_hs, xi_bs, xi_hs;            // coefficients of x; its intervals
    unsigned yw_bs, yw_hs, yi_bs, yi_hs;
    unsigned zw_bs, zw_hs;
    int heads, batches;
    int total_tiles;                                // batches * heads * D * (Lx / 128) * (Ly / 64)
    int dbg;
};

// Reduction lengths (in floats) the kernel is instantiated for.
inline bool dot_tiled_takes(int reduction) { return reduction == 32 || reduction == 64 || reduction == 128; }

// Floats of workspace the planes of one call need: |b| over the intervals of x, four planes over those of y.
inline long long dot_planes_floats(long long x_interval_floats, long long y_interval_floats) {
    return x_interval_floats + 4 * y_interval_floats;
}

// Writes the planes from the intervals (x_l: nx floats, y_l / y_u: ny floats; multiples of 4, 16-byte aligned).
void dot_planes_launch(const float *x_l, const float *y_l, const float *y_u, float *b_abs, float *al_pos, float *al_neg,
                       float *au_pos, float *au_neg, long long nx, long long ny, hipStream_t stream);

// vp: context path (y in its natural layout [k][m][j]).  grid: workgroups, a multiple of 8.
void dot_tiled_launch(bool vp, int reduction, const DotTiledArgs &a, int grid, hipStream_t stream);

}  // namespace faith

// The straight-line tiled kernel of the dot-product bounds (dot_tiled.hip) as dot.hip sees it.
#pragma once
#include "common.h"

namespace faith {

// Operands of one launch.  Every array is addressed through one buffer descriptor over the whole array and
// 32-bit byte offsets from its first element, so each array must span less than 4 GB (the entry point checks).
struct DotTiledArgs {
    const float *xlw, *xuw, *ylw, *yuw;             // coefficients
    const float *x_l, *y_l, *y_u;                   // concrete intervals: b = x_l, a_l = y_l, a_u = y_u
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
};

// Reduction lengths (in floats) the kernel is instantiated for.
inline bool dot_tiled_takes(int reduction) { return reduction == 32 || reduction == 64 || reduction == 128; }

// vp: context path (y in its natural layout [k][m][j]).  grid: workgroups, a multiple of 8.
void dot_tiled_launch(bool vp, int reduction, const DotTiledArgs &a, int grid, hipStream_t stream);

}  // namespace faith

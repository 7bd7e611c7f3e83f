// The MFMA kernels of the dot-product bounds in the reference's transposed layout (dot_transposed.hip) as dot.hip
// sees them.
#pragma once
#include "common.h"

namespace faith {

// Operands of the two launches (see dot_transposed.hip); every array as dot_entry_transposed has it.
struct DotTransposedArgs {
    const float *xlw, *xuw, *ylw, *yuw;   // [T, Lx, K, D], [T, Ly, K, D]
    const float *x_l, *y_l, *y_u;         // [T, Lx, K], [T, Ly, K]
    float *zlw, *zuw;                     // [T, Lx, Ly, D]
    int T, Lx, Ly, K, D;
};

// Whether the shape is one the kernels take (lengths in whole 32-row blocks, dim_in in whole 32-lane blocks, a
// reduction in chunks of 16, the intervals of one batch element within the LDS of two workgroups per CU).
bool dot_transposed_mfma_takes(int Lx, int Ly, int K, int D);

// Both launches on `stream`.  False if the device refused the LDS size (nothing launched).
bool dot_transposed_mfma_launch(const DotTransposedArgs &a, hipStream_t stream);

}  // namespace faith

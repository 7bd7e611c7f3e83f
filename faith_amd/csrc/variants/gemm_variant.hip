// One generated variant of the sign-split GEMM's MFMA kernel, compiled on request by faith_amd.autotune
// (generate -> compile -> measure -> keep the fastest: what the reference's autotuner does by rewriting
// matmul_config.h and rebuilding its extension, Transformer_Verification_Code/autotuner/).  The library ships four
// macro-tiles; this translation unit takes any tile shape the tile code can express and the scheduling switches as
// macros:
//
//   FAITH_V_MBM, FAITH_V_MBN   32 x 32 MFMA blocks per wavefront along M and N (macro-tile 64 MBM x 64 MBN;
//                              MBM * MBN <= 4: the accumulators are 32 MBM MBN registers)
//   FAITH_V_WAVES              wavefronts per SIMD the register budget is set for (1 ... 4)
//   FAITH_GEMM_SETPRIO         0 / 1: raised priority during a run of MFMAs (see gemm_tile.h)
//
// It serves the coefficient rows only ([rows, K] x [N, K]^T, the MFMA part, which is what a variant changes); the
// constant-term rows of a layer stay with the library's exact-accumulation kernel.  Built into a library of its own
// together with common.hip.
#include "../gemm_tile.h"

#if !defined(FAITH_V_MBM) || !defined(FAITH_V_MBN) || !defined(FAITH_V_WAVES)
#error "gemm_variant.hip is compiled with -DFAITH_V_MBM= -DFAITH_V_MBN= -DFAITH_V_WAVES="
#endif
static_assert(FAITH_V_MBM >= 1 && FAITH_V_MBN >= 1 && FAITH_V_MBM * FAITH_V_MBN <= 4, "at most 128 accumulator registers per operand");
static_assert(FAITH_V_WAVES >= 1 && FAITH_V_WAVES <= 4, "wavefronts per SIMD");

namespace {

constexpr int V_BM = 64 * FAITH_V_MBM, V_BN = 64 * FAITH_V_MBN;
constexpr size_t V_LDS = (size_t)2 * (4 * V_BM * 8 + 4 * V_BN * 8) * sizeof(float);     // two stages of four operand tiles
static_assert(V_LDS <= 160 * 1024, "the two LDS stages of this tile do not fit a workgroup");

template <bool EXACT>
__global__ void __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(FAITH_V_WAVES, FAITH_V_WAVES)))
variant_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) float sm[];
    signsplit_gemm_body<EXACT, FAITH_V_MBM, FAITH_V_MBN>(g, sm, blockIdx.x);
}

}  // namespace

extern "C" int faith_variant_lds_bytes(void) { return (int)V_LDS; }

// y_lw, y_uw [rows, dim_y_out] = sign-split product of x_lw, x_uw [rows, dim_out] with W [dim_y_out, dim_out]
// (Bounds.ori_matmul on the coefficient rows, Bounds.py:397-413).  FAITH_ERR_UNSUPPORTED for what the MFMA tile does
// not take (dim_out % 4 != 0, operands not 16-byte aligned, a tile's rows spanning 4 GB).
extern "C" int faith_variant_matmul_coefficients(const float *x_lw, const float *x_uw, const float *W, float *y_lw,
                                                 float *y_uw, long long rows, int dim_out, int dim_y_out, void *stream) {
    FAITH_NOT_NULL(x_lw); FAITH_NOT_NULL(x_uw); FAITH_NOT_NULL(W); FAITH_NOT_NULL(y_lw); FAITH_NOT_NULL(y_uw);
    FAITH_ALIGNED4(y_lw); FAITH_ALIGNED4(y_uw);
    FAITH_REQUIRE(rows > 0 && rows <= 0x7fffffffLL && dim_out > 0 && dim_y_out > 0, FAITH_ERR_SHAPE,
                  "faith_variant_matmul_coefficients: rows=%lld dim_out=%d dim_y_out=%d must be positive", rows, dim_out, dim_y_out);
    FAITH_REQUIRE(dim_out % 4 == 0 && faith::aligned(x_lw, 16) && faith::aligned(x_uw, 16) && faith::aligned(W, 16) &&
                      (long long)V_BM * dim_out * 4 < 0xffffffffLL && (long long)V_BN * dim_out * 4 < 0xffffffffLL &&
                      (long long)V_BM * dim_y_out * 4 < 0x80000000LL,
                  FAITH_ERR_UNSUPPORTED,
                  "faith_variant_matmul_coefficients: needs dim_out %% 4 == 0, 16-byte aligned operands and tiles under 4 GB");
    GemmArgs g{};
    g.Al = x_lw; g.Au = x_uw; g.W = W; g.Cl = y_lw; g.Cu = y_uw;
    g.Mw = (int)rows; g.Mb = 0; g.N = dim_y_out; g.K = dim_out;
    const long long mblks = (rows + V_BM - 1) / V_BM;
    const long long grid = ((mblks + XCDS - 1) / XCDS) * XCDS * ((dim_y_out + V_BN - 1) / V_BN);
    FAITH_REQUIRE(grid <= 0x7fffffffLL, FAITH_ERR_SHAPE, "faith_variant_matmul_coefficients: grid too large");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dim_out % BK == 0) {
        FAITH_REQUIRE(faith::reserve_lds(variant_kernel<true>, V_LDS), FAITH_ERR_UNSUPPORTED, "faith_variant_matmul_coefficients: LDS");
        hipLaunchKernelGGL(variant_kernel<true>, dim3((unsigned)grid), dim3(NTHREADS), V_LDS, st, g);
    } else {
        FAITH_REQUIRE(faith::reserve_lds(variant_kernel<false>, V_LDS), FAITH_ERR_UNSUPPORTED, "faith_variant_matmul_coefficients: LDS");
        hipLaunchKernelGGL(variant_kernel<false>, dim3((unsigned)grid), dim3(NTHREADS), V_LDS, st, g);
    }
    return faith::check_launch("faith_variant_matmul_coefficients");
}

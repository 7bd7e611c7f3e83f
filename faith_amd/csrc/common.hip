// Error bookkeeping of the C ABI (no kernels here).
#include "common.h"

namespace faith {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: HIP error %d (%s)", what, static_cast<int>(e), hipGetErrorString(e));
        return FAITH_ERR_LAUNCH;
    }
    return FAITH_OK;
}

bool dual_exponent(int q, float *qv) {
    if (q == FAITH_Q_1 || q == FAITH_Q_2 || q == FAITH_Q_INF) return true;
    float f;
    static_assert(sizeof(f) == sizeof(q), "q carries the bits of a float");
    __builtin_memcpy(&f, &q, sizeof(f));
    if (!(f > 1.0f) || f > 3.0e38f) return false;      // rejects NaN, inf, and anything <= 1
    *qv = f;
    return true;
}

int compute_units() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// per calling thread: a tuning table applied around one thread's launch does not steer another thread's
static thread_local int g_tune[FAITH_TUNE_COUNT] = {0};

int tune_get(int knob) { return (knob >= 0 && knob < FAITH_TUNE_COUNT) ? g_tune[knob] : 0; }

}  // namespace faith

extern "C" int faith_tune_set(int knob, int value) {
    if (knob < 0 || knob >= FAITH_TUNE_COUNT) {
        faith::set_error("faith_tune_set: unknown knob %d", knob);
        return FAITH_ERR_UNSUPPORTED;
    }
    faith::g_tune[knob] = value;
    return FAITH_OK;
}

// Plain streaming copy: the yardstick the HBM-bound kernels are compared with, and the kernel
// of known size that hardware byte counters are calibrated against.
__global__ void __launch_bounds__(256) copy_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst,
                                                   size_t n4) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

extern "C" int faith_copy_f32(const float *src, float *dst, long long n, void *stream) {
    FAITH_NOT_NULL(src);
    FAITH_NOT_NULL(dst);
    FAITH_REQUIRE(n > 0 && n % 4 == 0, FAITH_ERR_SHAPE, "faith_copy_f32: n=%lld must be a positive multiple of 4", n);
    FAITH_REQUIRE(faith::aligned(src, 16) && faith::aligned(dst, 16), FAITH_ERR_ALIGN,
                  "faith_copy_f32: pointers must be 16-byte aligned");
    const size_t n4 = (size_t)n / 4;
    const unsigned blocks = (unsigned)((n4 + 255) / 256 < 256 * 32 ? (n4 + 255) / 256 : 256 * 32);
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<const float4 *>(src), reinterpret_cast<float4 *>(dst), n4);
    return faith::check_launch("faith_copy_f32");
}

// Shader clock under matrix load: every workgroup keeps its four SIMDs issuing fp32 MFMAs for
// `iterations` rounds of 16 and divides the shader-cycle counter by the constant 100 MHz counter.
typedef float clk_floatx16 __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256) mfma_clock_kernel(float *__restrict__ mhz, const int iterations) {
    clk_floatx16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    const float a = 1e-3f * (float)(threadIdx.x % 7), b = 0.5f;
    const unsigned long long c0 = __builtin_readcyclecounter();
    const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
    float keep = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) keep += acc[i][0];
    if (threadIdx.x == 0)
        mhz[blockIdx.x] = (r1 > r0 ? (float)((double)(c1 - c0) / (double)(r1 - r0) * 100.0) : 0.f) + (keep == 1234.5f ? 1.f : 0.f);
}

extern "C" int faith_mfma_clock(float *mhz, int workgroups, int iterations, void *stream) {
    FAITH_NOT_NULL(mhz);
    FAITH_REQUIRE(workgroups > 0 && workgroups <= 65536 && iterations > 0 && iterations <= 100000, FAITH_ERR_SHAPE,
                  "faith_mfma_clock: workgroups=%d (1..65536), iterations=%d (1..100000)", workgroups, iterations);
    hipLaunchKernelGGL(mfma_clock_kernel, dim3((unsigned)workgroups), dim3(256), 0, static_cast<hipStream_t>(stream), mhz,
                       iterations);
    return faith::check_launch("faith_mfma_clock");
}

extern "C" const char *faith_last_error(void) { return faith::g_error; }

// 2: faith_dot_product_verification_QK / _V take `int layout` in front of `stream` (version 1 did not).
extern "C" int faith_version(void) { return 2; }

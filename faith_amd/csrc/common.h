// Shared host-side helpers of the C ABI: status codes, error text, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/faith_amd.h"

namespace faith {

// Thread-local message behind faith_last_error().
void set_error(const char *fmt, ...);

// Returns FAITH_OK or records the HIP error text and returns FAITH_ERR_LAUNCH.
int check_launch(const char *what);

// One-launch concretization of two bound objects of one dim_in (defined with the relaxation kernels); rows2 == 0:
// of one.  `u` may be NULL (the upper interval of the first object is not wanted): its upper coefficients are
// then not read in the natural layout.
int concretize_pair(const float *lb, const float *ub, const float *lw, const float *uw, float *l, float *u, int rows,
                    const float *lb2, const float *ub2, const float *lw2, const float *uw2, float *l2, float *u2,
                    int rows2, int dim_in, int dim_out, int dim_out2, float eps, int q, int words, void *stream,
                    int layout = FAITH_LAYOUT_NATURAL);

// The `q` argument of the entry points: FAITH_Q_1 / FAITH_Q_2 / FAITH_Q_INF, or the IEEE-754 bits of any
// other dual exponent in (1, inf) (written to *qv).  False if it is neither.
bool dual_exponent(int q, float *qv);

// Compute units of the current device (queried once per device, then cached).
int compute_units();

// Tuning knobs (faith_tune_set); 0 = built-in choice.
int tune_get(int knob);

// A launch that asks for more than 64 KB of dynamic LDS has to raise the kernel's limit first (160 KB per
// workgroup on this part).  False if the request cannot be met; a launch that follows a false return fails
// and is reported by check_launch.
template <typename Kernel>
inline bool reserve_lds(Kernel kernel, size_t bytes) {
    if (bytes <= 64 * 1024) return true;
    if (bytes > 160 * 1024) return false;
    return hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               static_cast<int>(bytes)) == hipSuccess;
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline int ceil_div(long long a, long long b) { return static_cast<int>((a + b - 1) / b); }

}  // namespace faith

#define FAITH_REQUIRE(cond, code, ...)      \
    do {                                    \
        if (!(cond)) {                      \
            faith::set_error(__VA_ARGS__);  \
            return (code);                  \
        }                                   \
    } while (0)

#define FAITH_NOT_NULL(p) FAITH_REQUIRE((p) != nullptr, FAITH_ERR_NULL, "%s: argument '%s' is NULL", __func__, #p)
#define FAITH_ALIGNED4(p) \
    FAITH_REQUIRE(faith::aligned((p), 4), FAITH_ERR_ALIGN, "%s: argument '%s' is not 4-byte aligned", __func__, #p)

// Shared helpers for the C-ABI implementation: error recording and launch
// checks. Nothing here crosses the ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "pet_hip.h"

namespace pet {

// Last error text, per host thread.
char *err_buf();
int set_error(int status, const char *fmt, ...);
bool initialised();
// Whether split contractions must add their partial sums in a fixed order.
bool deterministic();
// Split-K scratch owned by the library (see runtime.hip).
void splitk_workspace(float **ws, size_t *ws_elems, int **counters, int *num_counters);

#define PET_HIP_CHECK(expr)                                                    \
    do {                                                                       \
        hipError_t _e = (expr);                                                \
        if (_e != hipSuccess)                                                  \
            return pet::set_error(PET_HIP_ERR_RUNTIME, "%s failed: %s (%s:%d)", \
                                  #expr, hipGetErrorString(_e), __FILE__,      \
                                  __LINE__);                                   \
    } while (0)

#define PET_REQUIRE_INIT()                                                     \
    do {                                                                       \
        if (!pet::initialised())                                               \
            return pet::set_error(PET_HIP_ERR_NOT_INIT,                        \
                                  "pet_hip_init has not been called");         \
    } while (0)

// Checks the launch that was just issued. Under stream capture
// hipGetLastError still reports configuration errors.
inline int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return set_error(PET_HIP_ERR_RUNTIME, "launch of %s failed: %s", what,
                         hipGetErrorString(e));
    return PET_HIP_OK;
}

inline hipStream_t as_stream(pet_hip_stream_t s) { return (hipStream_t)s; }

__device__ __forceinline__ float apply_act(float v, int act) {
    switch (act) {
    case PET_HIP_ACT_RELU:
        return v > 0.f ? v : 0.f;
    case PET_HIP_ACT_SIGMOID:
        return 1.f / (1.f + expf(-v));
    case PET_HIP_ACT_TANH:
        return tanhf(v);
    case PET_HIP_ACT_GELU:
        return 0.5f * v * (1.f + erff(v * 0.70710678118654752440f));
    default:
        return v;
    }
}

} // namespace pet

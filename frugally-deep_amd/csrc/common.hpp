// Shared host/device helpers of the fdx library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/fdx.h"

namespace fdx {

// thread-local error text behind fdx_last_error()
void set_error(const char* fmt, ...);
hipStream_t stream();
bool profiling();
// records one launch for the per-kernel profile (flops / bytes are algorithmic figures)
void profile_begin();
void profile_end(const char* family, double flops, double bytes);

struct Act {
    int kind;
    float max_value, negative_slope, threshold;
};

inline Act make_act(const fdx_act* a)
{
    Act r { FDX_ACT_NONE, 3.402823466e+38f, 0.f, 0.f };
    if (a) {
        r.kind = a->kind;
        r.max_value = a->max_value;
        r.negative_slope = a->negative_slope;
        r.threshold = a->threshold;
    }
    return r;
}

// include/fdeep/layers/relu_layer.hpp:40-46 and include/fdeep/recurrent_ops.hpp:73-76
__device__ __forceinline__ float apply_act(float x, const Act& a)
{
    if (a.kind == FDX_ACT_RELU) {
        if (x >= a.max_value)
            return a.max_value;
        if (x >= a.threshold)
            return x;
        return a.negative_slope * (x - a.threshold);
    }
    if (a.kind == FDX_ACT_GELU)
        return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f));
    return x;
}

} // namespace fdx

#define FDX_HIP(expr)                                                                                     \
    do {                                                                                                  \
        hipError_t e_ = (expr);                                                                           \
        if (e_ != hipSuccess) {                                                                           \
            fdx::set_error("HIP error %s at %s:%d: %s", hipGetErrorName(e_), __FILE__, __LINE__, #expr);  \
            return FDX_ERR_HIP;                                                                           \
        }                                                                                                 \
    } while (0)

#define FDX_REQUIRE(cond, ...)                                                                            \
    do {                                                                                                  \
        if (!(cond)) {                                                                                    \
            fdx::set_error(__VA_ARGS__);                                                                  \
            return FDX_ERR_INVALID;                                                                       \
        }                                                                                                 \
    } while (0)

#define FDX_LAUNCH_CHECK()                                                                                \
    do {                                                                                                  \
        hipError_t e_ = hipGetLastError();                                                                \
        if (e_ != hipSuccess) {                                                                           \
            fdx::set_error("kernel launch failed (%s) at %s:%d", hipGetErrorName(e_), __FILE__, __LINE__);\
            return FDX_ERR_HIP;                                                                           \
        }                                                                                                 \
    } while (0)

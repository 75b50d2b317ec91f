// Shared host/device helpers of the fdx library (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "../../include/fdx.h"
#include "../../include/fdx_debug.h"

namespace fdx {

// thread-local error text behind fdx_last_error()
void set_error(const char* fmt, ...);
hipStream_t stream();
bool profiling();
// Clears library-owned scratch at set-up time, on the library stream (which does not synchronise with the null
// stream) and waits for it, so that the first kernel that reads the cells sees zeros.  Not for use inside a stream capture.
hipError_t zero_device(void* p, size_t bytes);
// pinned host int that kernels store a code to when a bounded wait runs out; fdx_sync and fdx_d2h report and clear it
int* async_error_cell();
// records one launch for the per-kernel profile (flops / bytes are algorithmic figures; executed_flops = the
// multiply-adds the kernel really issues where that differs, as in the Winograd form; negative = the same)
void profile_begin();
void profile_end(const char* family, double flops, double bytes, double executed_flops = -1.0);

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

// The same for a block of values, with the switch on the kind outside the element loop and a branch-free ReLU that
// keeps the order of the tests above (x >= max first, then x >= threshold).  Per element, apply_act's tests become
// exec-mask branches, which in a short kernel can cost more instructions than the arithmetic around them.
template <int COUNT>
__device__ __forceinline__ void apply_act_block(float (&v)[COUNT], const Act& a)
{
    if (a.kind == FDX_ACT_RELU) {
#pragma unroll
        for (int z = 0; z < COUNT; ++z) {
            const float x = v[z];
            const float low = x >= a.threshold ? x : a.negative_slope * (x - a.threshold);
            v[z] = x >= a.max_value ? a.max_value : low;
        }
    } else if (a.kind == FDX_ACT_GELU) {
#pragma unroll
        for (int z = 0; z < COUNT; ++z)
            v[z] = 0.5f * v[z] * (1.0f + erff(v[z] * 0.70710678118654752440f));
    }
}

// every activation kind (stand-alone activation kernel only; the epilogues keep the two-way switch above
// so that the GEMM kernels do not carry transcendental code they never run)
__device__ __forceinline__ float apply_act_full(float x, const Act& a)
{
    switch (a.kind) {
    case FDX_ACT_NONE: return x;
    case FDX_ACT_RELU:
    case FDX_ACT_GELU: return apply_act(x, a);
    case FDX_ACT_TANH: return tanhf(x);
    case FDX_ACT_SIGMOID: return 1.0f / (1.0f + expf(-x));
    case FDX_ACT_SWISH: return x / (1.0f + expf(-x));
    case FDX_ACT_HARD_SIGMOID: return x < -3.0f ? 0.0f : (x > 3.0f ? 1.0f : x / 6.0f + 0.5f);
    case FDX_ACT_SELU: return 1.0507009873554804934193349852946f * (x >= 0.0f ? x : 1.6732632423543772848170429916717f * (expf(x) - 1.0f));
    case FDX_ACT_ELU: return x >= 0.0f ? x : a.negative_slope * (expf(x) - 1.0f);
    case FDX_ACT_EXPONENTIAL: return expf(x);
    case FDX_ACT_SOFTSIGN: return x / (fabsf(x) + 1.0f);
    case FDX_ACT_SOFTPLUS: {
        const float thr = -13.942385f; // log(FLT_EPSILON) + 2
        return x > -thr ? x : (x < thr ? expf(x) : log1pf(expf(x)));
    }
    case FDX_ACT_LEAKY_RELU: return x > 0.0f ? x : a.negative_slope * x;
    case FDX_ACT_HARD_SHRINK: return fabsf(x) > a.threshold ? x : 0.0f;
    case FDX_ACT_SOFT_SHRINK: return x > a.threshold ? x - a.threshold : (x < -a.threshold ? x + a.threshold : 0.0f);
    case FDX_ACT_SPARSE_PLUS: return x <= -1.0f ? 0.0f : (x < 1.0f ? 0.25f * (x + 1.0f) * (x + 1.0f) : x);
    case FDX_ACT_SQUARE_PLUS: return (x + sqrtf(x * x + a.max_value)) / 2.0f;
    case FDX_ACT_TANH_SHRINK: return x - tanhf(x);
    case FDX_ACT_THRESHOLD: return x > a.threshold ? x : a.max_value;
    case FDX_ACT_LOG_SIGMOID: return logf(1.0f / (1.0f + expf(-x)));
    case FDX_ACT_HARD_TANH: return x < -1.0f ? -1.0f : (x > 1.0f ? 1.0f : x);
    case FDX_ACT_LOG: return logf(x);
    default: return x;
    }
}

// Sum over the sixteen lanes of a row (lanes 16r .. 16r+15), left in every lane of the row, on the VALU's data-parallel
// primitives: swaps inside quads, then the mirror inside each half row and inside the row (after the quad steps all lanes
// of a quad agree, so the mirrored partner holds the other quads' sum).  __shfl_xor compiles to ds_bpermute_b32, a trip
// through the LDS crossbar with an address register and a wait of its own per step.
#if defined(__HIPCC__) // device-only builtins; a plain host compiler (the sanitizer build of the loader) skips them
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row16_sum(float v)
{
    v += dpp_move<0xB1>(v);  // quad_perm [1, 0, 3, 2]
    v += dpp_move<0x4E>(v);  // quad_perm [2, 3, 0, 1]
    v += dpp_move<0x141>(v); // row_half_mirror
    v += dpp_move<0x140>(v); // row_mirror
    return v;
}
#endif

// activations an epilogue can carry
inline bool epilogue_act_ok(const fdx_act* a) { return !a || a->kind == FDX_ACT_NONE || a->kind == FDX_ACT_RELU || a->kind == FDX_ACT_GELU; }

} // namespace fdx

#define FDX_REQUIRE_EPILOGUE_ACT(act)                                                                     \
    do {                                                                                                  \
        if (!fdx::epilogue_act_ok(act)) {                                                                 \
            fdx::set_error("this launcher fuses only NONE / RELU / GELU; run other activations through fdx_activation_f32"); \
            return FDX_ERR_UNSUPPORTED;                                                                   \
        }                                                                                                 \
    } while (0)

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

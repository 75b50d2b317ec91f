// Decode attention for the common head shape (key_dim = value_dim = 64, at most 256 cached
// positions): one query row per (sequence, head) against the token-major key / value cache.
//
// The kernel is one memory round trip: every lane issues all of its key AND value loads
// (16 bytes each, sixteen lanes per cached row so a wave touches four whole rows per load)
// before anything is used; the values do not depend on the softmax, so they travel while the
// scores are reduced.  Scores stay in registers; max / sum / output reductions use wave
// shuffles and ONE small LDS exchange between the four waves.  Softmax weights equal the
// reference's exp(x - m - log(sum)) (include/fdeep/tensor.hpp:1165-1192) up to rounding; the
// scale multiplies the scores after the dot product (layers/multi_head_attention_layer.hpp:91-93).
#include <cfloat>
#include <cmath>

#include "common.hpp"
#include "global_ptr.hpp"
#include "skinny.hpp"

namespace fdx {

typedef float f32x4 __attribute__((ext_vector_type(4)));

#include "decode_attn_body.hpp"

__global__ __launch_bounds__(256) void mha_decode_fast_kernel(const float* __restrict__ q, int64_t ldq,
    const float* __restrict__ kc, const float* __restrict__ vc, float* __restrict__ out, int heads,
    const int* __restrict__ len_dev, int max_len, float scale)
{
    __shared__ MhaDecodeShared sh;
    mha_decode_fast_body<false>(q, ldq, kc, vc, out, heads, len_dev, max_len, scale, blockIdx.x, threadIdx.x, true, sh, [] {});
}

// ---- decode attention and the layer's output projection as ONE launch ----------------------------------------------
//
// out[b][:] = act(bias + residual[b][:] + sum_h o_h[b] * Wo_h), where o_h[b] is the attention output of head h
// (layers/multi_head_attention_layer.hpp:74-95) and Wo_h the 64 rows of the output kernel that multiply head h's
// slice of the concatenated heads (same file :108-109: Dense over the heads concatenated in head order).
//
// A decode step is a chain of dependent launches, each a few microseconds of latency whatever it computes, so a
// launch saved is worth more than the extra bytes this form moves.  Workgroup (b, h) computes o_h[b] as the attention
// kernel does, keeps it in LDS, multiplies it by its head's slice of the kernel -- re-laid once per session as
// [head][64][output column] (the order the file stores it in), a contiguous 64 * n_out floats per head, which the sixteen workgroups of a head share
// through L2 -- and leaves its n_out partial sums in a workspace.  The heads of a sequence are then added by whichever
// of its workgroups finishes last: partials are written with agent-scope (write-through) stores and waited for
// (s_waitcnt vmcnt(0) behind a workgroup barrier) before one thread takes the sequence's ticket with an agent-scope
// atomic; the workgroup that draws the last ticket reads all partials with agent-scope loads, adds them IN HEAD ORDER
// (the sum does not depend on who arrives when), applies bias, residual and activation and writes the row.  Nobody waits
// for anybody.  Why the exchange is sound without cache-wide fences: an agent-scope store is complete, for the
// s_waitcnt that follows it, only once it has been written through to memory, the point where the XCDs' L2 caches
// meet; the ticket is taken after every thread's wait, so no ticket can be observed before the partials it covers; the
// last arriver's agent-scope loads are issued after its ticket returned and are served from that same point, never from
// a line its own L2 may hold.  This is what a release / acquire pair at agent scope does, restricted to the lines concerned.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
constexpr int kProjMaxOut = 1024; // output columns the kernel covers: four per thread
constexpr int kAgentScope = 16;   // cache-policy bit of a buffer access that makes it an agent-scope (write-through / re-fetched) one

__global__ __launch_bounds__(256) void mha_decode_proj_kernel(const float* __restrict__ q, int64_t ldq,
    const float* __restrict__ kc, const float* __restrict__ vc, int heads, const int* __restrict__ len_dev, int max_len,
    float scale, const float* __restrict__ wt, const float* __restrict__ bias, const float* __restrict__ residual, int64_t ldr,
    Act act, int n_out, float* __restrict__ workspace, int* __restrict__ tickets, float* __restrict__ out)
{
    __shared__ MhaDecodeShared sh;
    __shared__ int is_last;
    const int item = blockIdx.x, tid = threadIdx.x;
    const int b = item / heads, h = item % heads;
    // Thread t owns output columns 4t .. 4t+3: partial[n] = sum_d o[d] * wt[h][d][n], one 16-byte load per d, a wave reads a
    // contiguous kilobyte, no cross-lane reduction.  The head's slice of the kernel does not depend on the attention
    // result: the rows of the first sixteen d are requested right behind the key / value loads.
    const int n4 = tid * 4;
    const bool col_ok = n4 < n_out;
    const gptr<const float> wbase = as_global(wt) + ((int64_t)h * 64) * n_out + (col_ok ? n4 : 0);
    constexpr int ROUND = 32; // rows of the slice requested together (two rounds)
    f32x4 w[ROUND];
    auto load_rows = [&](int d0) {
#pragma unroll
        for (int u = 0; u < ROUND; ++u) {
            w[u] = f32x4 { 0.f, 0.f, 0.f, 0.f };
            if (col_ok)
                w[u] = *reinterpret_cast<gptr<const f32x4>>(wbase + (int64_t)(d0 + u) * n_out);
        }
    };
    mha_decode_fast_body<true>(q, ldq, kc, vc, nullptr, heads, len_dev, max_len, scale, item, tid, true, sh, [&] { load_rows(0); });
    __syncthreads();
    f32x4 acc = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
    for (int d0 = 0; d0 < 64; d0 += ROUND) {
        f32x4 cur[ROUND];
#pragma unroll
        for (int u = 0; u < ROUND; ++u)
            cur[u] = w[u];
        if (d0 + ROUND < 64)
            load_rows(d0 + ROUND); // in flight while this round is multiplied
#pragma unroll
        for (int u = 0; u < ROUND; ++u) {
            const float o = sh.oval[d0 + u];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc[e] += o * cur[u][e];
        }
    }
    // 16-byte agent-scope accesses through buffer resources: offsets beyond the extent drop the store / return zeros
    const int row_bytes = n_out * 4;
    const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(workspace + (int64_t)b * heads * n_out, 0,
        heads * row_bytes, 0x00020000);
    const int out_of_range = 0x7fffffff;
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc), ws_rsrc, col_ok ? h * row_bytes + n4 * 4 : out_of_range, 0,
        kAgentScope);
    // every lane's partials have been written through before the ticket is taken
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const gptr<int> ticket_cell = as_global(tickets) + b;
        const int ticket = __hip_atomic_fetch_add(ticket_cell, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = ticket == heads - 1;
        if (last)
            __hip_atomic_store(ticket_cell, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // for the next launch
        is_last = last;
    }
    __syncthreads();
    if (!is_last || !col_ok)
        return;
    // the partial rows of all heads are requested together, then added in head order
    f32x4 add = { 0.f, 0.f, 0.f, 0.f };
    if (bias)
        add = *reinterpret_cast<const f32x4*>(bias + n4);
    if (residual) {
        const f32x4 r = *reinterpret_cast<const f32x4*>(residual + (int64_t)b * ldr + n4);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            add[e] += r[e];
    }
    f32x4 v = { 0.f, 0.f, 0.f, 0.f };
    for (int h0 = 0; h0 < heads; h0 += 16) {
        f32x4 pv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u)
            pv[u] = __builtin_bit_cast(f32x4,
                __builtin_amdgcn_raw_buffer_load_b128(ws_rsrc, h0 + u < heads ? (h0 + u) * row_bytes + n4 * 4 : out_of_range, 0, kAgentScope));
#pragma unroll
        for (int u = 0; u < 16; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                v[e] += pv[u][e]; // rows beyond `heads` read as zeros
    }
    float r4[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        r4[e] = v[e] + add[e];
    apply_act_block<4>(r4, act);
    *reinterpret_cast<f32x4*>(out + (int64_t)b * n_out + n4) = f32x4 { r4[0], r4[1], r4[2], r4[3] };
}

// [n_out][heads * 64] (K contiguous, as the Dense launches read it) -> [heads][64][n_out], which is the order the
// file stores the kernel in: (heads, value_dim, output) (keras_export/convert_model.py:600-607)
__global__ __launch_bounds__(256) void pack_proj_heads_kernel(const float* __restrict__ w, int heads, int n_out, float* __restrict__ out)
{
    const int64_t total = (int64_t)heads * n_out * 64;
    for (int64_t z = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; z < total; z += (int64_t)gridDim.x * blockDim.x) {
        const int n = (int)(z % n_out), d = (int)((z / n_out) % 64), h = (int)(z / ((int64_t)64 * n_out));
        out[z] = w[(int64_t)n * heads * 64 + h * 64 + d];
    }
}

bool mha_decode_proj_supported(int batch, int heads, int dk, int dv, int max_len, int64_t ldq, int n_out, int64_t workspace_floats,
    int ticket_count)
{
    return dk == 64 && dv == 64 && max_len <= 256 && ldq % 4 == 0 && n_out > 0 && n_out <= kProjMaxOut && n_out % 4 == 0 && batch > 0
        && heads > 0 && (int64_t)batch * heads * n_out <= workspace_floats && batch <= ticket_count;
}

fdx_status pack_proj_heads_launch(const float* w_nk, int heads, int n_out, float* out)
{
    FDX_REQUIRE(w_nk && out && heads > 0 && n_out > 0, "pack_proj_heads: bad arguments");
    hipLaunchKernelGGL(pack_proj_heads_kernel, dim3(256), dim3(256), 0, stream(), w_nk, heads, n_out, out);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

fdx_status mha_decode_proj_launch(const float* q, int64_t ldq, const float* kc, const float* vc, int batch, int heads,
    const int* len_dev, int max_len, const float* wt, const float* bias, const float* residual, int64_t ldr, const Act& act, int n_out,
    float* workspace, int64_t workspace_floats, int* tickets, int ticket_count, float* out, int len_hint)
{
    FDX_REQUIRE(q && kc && vc && len_dev && wt && workspace && tickets && out, "mha_decode_proj: null pointer");
    FDX_REQUIRE(mha_decode_proj_supported(batch, heads, 64, 64, max_len, ldq, n_out, workspace_floats, ticket_count),
        "mha_decode_proj: shape outside the fused kernel's range");
    FDX_REQUIRE(!residual || residual != out, "mha_decode_proj: the residual must not alias the output");
    const float scale = (float)(1.0 / std::sqrt(64.0));
    profile_begin();
    FDX_REQUIRE(ldr % 4 == 0 && (reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(bias) | reinterpret_cast<uintptr_t>(residual)
                                    | reinterpret_cast<uintptr_t>(workspace)) % 16 == 0,
        "mha_decode_proj: 16-byte aligned operands required");
    hipLaunchKernelGGL(mha_decode_proj_kernel, dim3(batch * heads), dim3(256), 0, stream(), q, ldq, kc, vc, heads, len_dev, max_len,
        scale, wt, bias, residual, ldr, act, n_out, workspace, tickets, out);
    profile_end("mha_decode_proj_f32", 2.0 * batch * heads * (double)len_hint * 128 + 2.0 * batch * heads * 64.0 * n_out,
        4.0 * ((double)batch * len_hint * heads * 128 + (double)heads * 64 * n_out + 2.0 * batch * n_out));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

// true if the fast kernel covers this shape; launches it
bool mha_decode_fast_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch, int heads,
    int dk, int dv, const int* len_dev, int max_len, hipStream_t s)
{
    if (dk != 64 || dv != 64 || max_len > 256 || ldq % 4 != 0)
        return false;
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    hipLaunchKernelGGL(mha_decode_fast_kernel, dim3(batch * heads), dim3(256), 0, s, q, ldq, kc, vc, out, heads, len_dev, max_len, scale);
    return true;
}

} // namespace fdx

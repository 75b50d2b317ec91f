// Decode-shape kernels (gfx950): a handful of activation rows against a whole weight matrix.
//
// With at most 16 rows the GEMMs of a decode step are pure weight streaming: every byte of W
// is used once, so the kernel is HBM-bound and latency-bound, and the job is to put every
// load in flight at once and add nothing to the launch.  One workgroup of 8 wave64s owns 16
// output columns; the waves split K; each lane issues ALL its 16-byte weight and activation
// loads for a chunk of slabs before the first use, and v_mfma_f32_16x16x4_f32 does the 16x16
// products (it also performs the reduction along K that a VALU formulation would need
// cross-lane shuffles for).  The eight partial 16x16 tiles meet in LDS; bias, activation and
// residual are applied before the only store.
//
// A LayerNormalization in front of the GEMM costs no pass over the rows: with gamma folded
// into the weights (W' = W * gamma along k), their row sums s[n] and b' = b + W beta
// precomputed once, LN(x) W^T + b = rstd * (x W'^T - mean * s) + b', so the kernel multiplies
// the raw rows and only needs each row's mean and 1/sqrt(var + eps); both come from the
// activation registers the lanes already hold (two-pass variance, as the reference computes
// it) while the weight loads are still in flight.
//
// Up to three output segments let one launch write q and the new key / value cache rows.
#include <cfloat>
#include <cmath>
#include <cstdlib>
#include <cstring>

#include "common.hpp"
#include "global_ptr.hpp"
#include "skinny.hpp"

namespace fdx {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int SK_WAVES = 8;
constexpr int SK_CHUNK = 8;       // slabs of 16 k-values whose loads are issued together (8 waves x 8 x 16 = 1024 k)
constexpr int SK_CHUNK_LONG = 24; // long-K launches (up to 3072) still issue everything at once, one workgroup per CU

// SINGLE: the workgroup's K range fits one chunk per wave (only one register set is live, which
// triples the number of resident workgroups).  gridDim.y > 1 splits K across workgroups: partial
// tiles go to a workspace and the last workgroup to arrive at a column group (atomic ticket) adds
// them in split order -- deterministic, no spinning -- and runs the epilogue.
// LDS of one workgroup of the Dense kernel
struct SkinnyShared {
    float red[SK_WAVES * 256];
    int is_last;
    float stat[SK_WAVES * 16], stat2[SK_WAVES * 16]; // per-wave row sums / sums of squared deviations
};

// The work of workgroup (bx, by) of a (gx, gy) grid.
// EMB: the instantiation that knows the embedding prologue (SkinnyParams::emb_x / emb_res); the others carry none of its code
template <int CHUNK, bool SINGLE, bool EMB = false>
__device__ __forceinline__ void skinny_gemm_body(const SkinnyParams& p, int bx, int by, int gx, int gy, SkinnyShared& sh)
{
    float* red = sh.red;
    float* stat = sh.stat;
    float* stat2 = sh.stat2;
    int& is_last = sh.is_last;
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int i = lane & 15, kq = lane >> 4;
    const int n0 = bx * 16;
    const int K = p.K;

    // K range of this workgroup (split index by) and of this wave, multiples of 16
    const int ksplit = gy;
    const int per_wg = ((K + ksplit * 16 - 1) / (ksplit * 16)) * 16;
    const int wg_begin = by * per_wg;
    const int wg_end = wg_begin + per_wg < K ? wg_begin + per_wg : K;
    const int per_wave = ((per_wg + SK_WAVES * 16 - 1) / (SK_WAVES * 16)) * 16;
    const int k_begin = wg_begin + wave * per_wave;
    const int k_end = k_begin + per_wave < wg_end ? k_begin + per_wave : wg_end;
    const int slabs = k_end > k_begin ? (k_end - k_begin + 15) / 16 : 0;

    const int n = n0 + i;
    const bool n_ok = n < p.N, m_ok = i < p.M;
    const gptr<const float> Wg = as_global(p.W);
    const gptr<const float> wrow = Wg + (int64_t)(n_ok ? n : 0) * p.ldw;
    const int spw = per_wave / 16; // slabs per wave in the packed layout
    const bool emb = EMB && p.emb_x != 0;
    const bool emb_res = EMB && p.emb_res != 0;
    // embedding rows of this lane's activation row: token id (a float in the model's input) and position, both checked
    const int emb_pos = (emb || emb_res) ? *as_global(p.len_dev) : 0;
    auto emb_row = [&](int row, bool& ok) -> int64_t {
        const float f = as_global(p.emb_ids)[row];
        const int64_t id = (f >= 0.f && f < 9.0e18f) ? (int64_t)f : -1;
        ok = id >= 0 && id < p.emb_a_rows && emb_pos < p.emb_b_rows;
        return ok ? id : 0;
    };
    bool emb_ok = true;
    const int64_t emb_id = emb && m_ok ? emb_row(i, emb_ok) : 0;
    if (emb && m_ok && !emb_ok && p.emb_err && bx == 0 && by == 0 && wave == 0 && kq == 0)
        atomicExch(p.emb_err, 1);
    const gptr<const float> xrow = emb ? as_global(p.emb_a) + emb_id * K : as_global(p.X) + (int64_t)(m_ok ? i : 0) * p.ldx;
    const gptr<const float> xrow_b = emb ? as_global(p.emb_b) + (int64_t)(emb_ok ? emb_pos : 0) * K : xrow;
    // two named register sets (indexing one array with a run-time buffer number would push it to scratch)
    f32x4 w0[CHUNK], a0[CHUNK];
    auto load_chunk = [&](f32x4 (&wreg)[CHUNK], f32x4 (&areg)[CHUNK], int s0) {
#pragma unroll
        for (int s = 0; s < CHUNK; ++s) {
            const int k = k_begin + (s0 + s) * 16 + kq * 4;
            const bool k_ok = s0 + s < slabs && k < k_end;
            f32x4 wv = { 0.f, 0.f, 0.f, 0.f }, av = { 0.f, 0.f, 0.f, 0.f };
            if (p.packed) {
                // pre-packed operand: this wave's slab is one contiguous 1 KB run, zeros baked in
                if (s0 + s < spw)
                    wv = __builtin_nontemporal_load(reinterpret_cast<gptr<const f32x4>>(Wg) + (((int64_t)bx * SK_WAVES + wave) * spw + (s0 + s)) * 64 + lane);
            } else if (n_ok && k_ok)
                wv = __builtin_nontemporal_load(reinterpret_cast<gptr<const f32x4>>(wrow + k)); // every weight is used once per launch
            if (m_ok && k_ok) {
                av = *reinterpret_cast<gptr<const f32x4>>(xrow + k);
                if (emb) {
                    const f32x4 bv = *reinterpret_cast<gptr<const f32x4>>(xrow_b + k);
                    av = emb_ok ? av + bv : f32x4 { 0.f, 0.f, 0.f, 0.f };
                }
            }
            wreg[s] = wv;
            areg[s] = av;
        }
    };
    load_chunk(w0, a0, 0);

    // epilogue operands of this thread's output element travel with the weights instead of costing a
    // second dependent round trip after the reduction
    const int em = t >> 4, ecol = n0 + (t & 15);
    const bool e_ok = t < 256 && em < p.M && ecol < p.N;
    float e_bias = 0.f, e_res = 0.f, e_wsum = 0.f;
    int64_t e_shift = 0;
    int e_seg = 0;
    if (e_ok) {
        if (p.bias)
            e_bias = as_global(p.bias)[ecol];
        if (emb_res) {
            bool ok = true;
            const int64_t id = emb_row(em, ok);
            e_res = ok ? as_global(p.emb_a)[id * p.N + ecol] + as_global(p.emb_b)[(int64_t)emb_pos * p.N + ecol] : 0.f;
        } else if (p.residual)
            e_res = as_global(p.residual)[(int64_t)em * p.ldr + ecol];
        if (p.ln)
            e_wsum = as_global(p.w_rowsum)[ecol];
        if (p.n_seg > 1 && ecol >= p.seg[1].col_begin)
            e_seg = 1;
        if (p.n_seg > 2 && ecol >= p.seg[2].col_begin)
            e_seg = 2;
        if (p.seg[e_seg].len_stride)
            e_shift = (int64_t)(*as_global(p.len_dev)) * p.seg[e_seg].len_stride;
    }

    // 16x16x4 MFMA: A operand lane (m = i, k slot = kq), B operand lane (n = i, k slot = kq);
    // lane l ends up with D[4*(l/16) + e][l%16], e = 0..3.
    f32x4 acc = { 0.f, 0.f, 0.f, 0.f };
    auto compute_chunk = [&](const f32x4 (&wreg)[CHUNK], const f32x4 (&areg)[CHUNK]) {
#pragma unroll
        for (int s = 0; s < CHUNK; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(areg[s][e], wreg[s][e], acc, 0, 0, 0);
    };

    if (p.ln) {
        // rows fit one chunk (host guarantees K <= 8 * CHUNK * 16): statistics from the registers
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < CHUNK; ++c)
            s += (a0[c][0] + a0[c][1]) + (a0[c][2] + a0[c][3]);
        s += __shfl_xor(s, 16, 64);
        s += __shfl_xor(s, 32, 64);
        if (kq == 0)
            stat[wave * 16 + i] = s;
        __syncthreads();
        // every thread adds the eight partial sums of its row itself (same order everywhere, so the same value): the
        // mean costs this one barrier, and the squared deviations ride on the barrier of the product reduction
        float tot = 0.f;
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w)
            tot += stat[w * 16 + i];
        const float mean = tot / (float)K;
        float q = 0.f;
#pragma unroll
        for (int c = 0; c < CHUNK; ++c) {
            const int k = k_begin + c * 16 + kq * 4;
            if (c < slabs && k < k_end) { // padding lanes hold zeros, not row values
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float d = a0[c][e] - mean;
                    q += d * d;
                }
            }
        }
        q += __shfl_xor(q, 16, 64);
        q += __shfl_xor(q, 32, 64);
        if (kq == 0)
            stat2[wave * 16 + i] = q;
        compute_chunk(w0, a0);
    } else if (SINGLE) {
        compute_chunk(w0, a0);
    } else {
        f32x4 w1[CHUNK], a1[CHUNK];
        for (int s0 = 0; s0 < slabs; s0 += 2 * CHUNK) {
            if (s0 + CHUNK < slabs)
                load_chunk(w1, a1, s0 + CHUNK);
            compute_chunk(w0, a0);
            if (s0 + 2 * CHUNK < slabs)
                load_chunk(w0, a0, s0 + 2 * CHUNK);
            if (s0 + CHUNK < slabs)
                compute_chunk(w1, a1);
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
        red[wave * 256 + (4 * kq + e) * 16 + i] = acc[e];
    __syncthreads();
    float v = 0.f;
    if (t < 256) {
#pragma unroll
        for (int w = 0; w < SK_WAVES; ++w)
            v += red[w * 256 + t];
    }
    if (ksplit > 1 && p.local_split) {
        // All K ranges of this column group run on one XCD (see SkinnyParams::local_split): partial tiles, flags and the
        // final sum go through that XCD's L2 with group-scope accesses (they miss the CU's own cache and are served by
        // the L2 the writers wrote through to), which costs a third of the exchange through memory below.  The last K
        // range is the one that waits: workgroups start in the order of their linear index, so everything it waits for
        // is already running or done, whatever else occupies the chip.
        constexpr int kGroup = 1, kDevice = 16; // cache-policy bits of a buffer access: sc0 = group scope, sc1 = device scope
        const int n_flags = p.ticket_count / 2;
        const __amdgpu_buffer_rsrc_t ws_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.workspace, 0, (int)((int64_t)gx * ksplit * 1024), 0x00020000);
        const __amdgpu_buffer_rsrc_t fl_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.tickets + n_flags, 0, n_flags * 4, 0x00020000);
        const unsigned xcc = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u; // XCC_ID: which XCD this workgroup runs on
        if (by != ksplit - 1) {
            if (t < 256)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), ws_rsrc, ((by * gx + bx) * 256 + t) * 4, 0, kGroup);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (t == 0)
                __builtin_amdgcn_raw_buffer_store_b32(1u + xcc, fl_rsrc, (bx * 8 + by) * 4, 0, kGroup);
            return;
        }
        if (t < ksplit - 1) {
            unsigned f = 0;
            for (int spin = 0; spin < (1 << 18); ++spin) {
                // Device scope for the flag: a group-scope load may be answered by this CU's own cache, which keeps the
                // zero it saw first (measured: such polls never saw the flag); the line lies in this XCD's L2 either way.
                // The compiler barriers keep the load inside the loop (as a read-only intrinsic it would be hoisted).
                asm volatile("" ::: "memory");
                f = __builtin_amdgcn_raw_buffer_load_b32(fl_rsrc, (bx * 8 + t) * 4, 0, kDevice);
                asm volatile("" ::: "memory");
                if (f)
                    break;
                __builtin_amdgcn_s_sleep(1);
            }
            if (f != 1u + xcc && p.err)
                __hip_atomic_store(p.err, (int)(kErrSplitExchange | (f << 8) | (xcc << 16) | ((unsigned)t << 24)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        __syncthreads();
        if (t < 256) {
            float pv[8];
#pragma unroll
            for (int ks = 0; ks < 7; ++ks)
                pv[ks] = ks < ksplit - 1
                    ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ws_rsrc, ((ks * gx + bx) * 256 + t) * 4, 0, kGroup))
                    : 0.f;
            const float own = v;
            v = 0.f;
#pragma unroll
            for (int ks = 0; ks < 7; ++ks)
                if (ks < ksplit - 1)
                    v += pv[ks];
            v += own;
        }
        if (t < ksplit - 1)
            __builtin_amdgcn_raw_buffer_store_b32(0u, fl_rsrc, (bx * 8 + t) * 4, 0, kGroup); // for the next launch
    } else if (ksplit > 1) {
        // Publish this split's partial tile with device-scope stores (they go past the XCD's L2), wait for
        // them, then take a ticket; only the last arrival continues and adds the partials in split order,
        // which makes the sum independent of arrival order.  No fence that writes back the whole L2.
        const gptr<float> ws = as_global(p.workspace);
        const gptr<int> tickets = as_global(p.tickets);
        const gptr<float> part = ws + ((int64_t)by * gx + bx) * 256;
        if (t < 256)
            __hip_atomic_store(part + t, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // every lane's partials have left the CU before the ticket is taken
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (t == 0) {
            const int ticket = __hip_atomic_fetch_add(tickets + bx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = ticket == ksplit - 1;
            if (is_last)
                __hip_atomic_store(tickets + bx, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // next launch
        }
        __syncthreads();
        if (!is_last)
            return;
        if (t < 256) {
            // all partials are requested before the first is used (a loop of load-and-add would pay one round trip to
            // memory per K range), then added in split order
            float pv[8];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
                pv[ks] = ks < ksplit ? __hip_atomic_load(ws + ((int64_t)ks * gx + bx) * 256 + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
            v = 0.f;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks)
                if (ks < ksplit)
                    v += pv[ks];
        }
    }
    if (e_ok) {
        if (p.ln) {
            float tot = 0.f, dev = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w) {
                tot += stat[w * 16 + em];
                dev += stat2[w * 16 + em];
            }
            v = (1.0f / sqrtf(dev / (float)K + p.ln_eps)) * (v - (tot / (float)K) * e_wsum);
        }
        v = apply_act(v + e_bias + e_res, p.act);
        const SkinnySegment& sg = p.seg[e_seg];
        const gptr<float> dst = as_global(sg.ptr) + e_shift + (int64_t)em * sg.ld + (ecol - sg.col_begin);
        *dst = v;
    }
}

template <int CHUNK, bool SINGLE, bool EMB = false>
__global__ __launch_bounds__(512) void skinny_gemm_kernel(SkinnyParams p)
{
    __shared__ SkinnyShared sh;
    skinny_gemm_body<CHUNK, SINGLE, EMB>(p, blockIdx.x, blockIdx.y, gridDim.x, gridDim.y, sh);
}


__device__ __forceinline__ unsigned long long pack_max(float v, int col);

// Wide outputs (a vocabulary projection: thousands of 16-column groups, K <= 1024): one workgroup per column
// group would run the chip in rounds, each paying the full load -> multiply -> reduce -> store latency chain with
// little in flight.  Here a fixed set of resident workgroups strides through the column groups: the activation
// rows (and the LayerNorm statistics) are taken once, and while one group's products are reduced and stored the next
// group's weights -- and its bias / residual / row-sum operands -- are already on their way in a second register set.
// (second bound: four waves per SIMD, i.e. two of these workgroups per CU)
template <int CHUNK>
__global__ __launch_bounds__(512, 4) void skinny_wide_kernel(SkinnyParams p, int tiles)
{
    // two reduction buffers taken in turn: a column group's partial tiles are summed out of one while the next group's go
    // into the other, so one barrier per group is enough (the barrier of group g + 1 orders every read of group g's
    // buffer before the writes of group g + 2)
    __shared__ float red_both[2][SK_WAVES * 256];
    __shared__ float stat[SK_WAVES * 16];
    __shared__ float row_mean[16], row_rstd[16];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int i = lane & 15, kq = lane >> 4;
    const int K = p.K;
    const int per_wave = ((K + SK_WAVES * 16 - 1) / (SK_WAVES * 16)) * 16;
    const int k_begin = wave * per_wave;
    const int k_end = k_begin + per_wave < K ? k_begin + per_wave : K;
    const int slabs = k_end > k_begin ? (k_end - k_begin + 15) / 16 : 0;
    const int spw = per_wave / 16;
    const bool m_ok = i < p.M;

    f32x4 a0[CHUNK];
    {
        const float* xrow = p.X + (int64_t)(m_ok ? i : 0) * p.ldx;
#pragma unroll
        for (int s = 0; s < CHUNK; ++s) {
            const int k = k_begin + s * 16 + kq * 4;
            a0[s] = (m_ok && s < slabs && k < k_end) ? *reinterpret_cast<const f32x4*>(xrow + k) : f32x4 { 0.f, 0.f, 0.f, 0.f };
        }
    }
    auto load_w = [&](f32x4 (&wreg)[CHUNK], int tile) {
        const int n = tile * 16 + i;
        const bool n_ok = n < p.N;
        const float* wrow = p.W + (int64_t)(n_ok ? n : 0) * p.ldw;
#pragma unroll
        for (int s = 0; s < CHUNK; ++s) {
            const int k = k_begin + s * 16 + kq * 4;
            f32x4 wv = { 0.f, 0.f, 0.f, 0.f };
            if (p.packed) {
                if (s < spw)
                    wv = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p.W) + (((int64_t)tile * SK_WAVES + wave) * spw + s) * 64 + lane);
            } else if (n_ok && s < slabs && k < k_end)
                wv = *reinterpret_cast<const f32x4*>(wrow + k); // 64-byte pieces of a row: the other half of the line is the next slab's
            wreg[s] = wv;
        }
    };
    // epilogue operands of output element (row em, column tile * 16 + ec), fetched with the tile's weights
    const int em = t >> 4, ec = t & 15;
    struct Epi {
        float bias, res, wsum;
    };
    auto load_epi = [&](int tile) {
        Epi e { 0.f, 0.f, 0.f };
        const int col = tile * 16 + ec;
        if (t < 256 && em < p.M && col < p.N) {
            if (p.bias)
                e.bias = p.bias[col];
            if (p.residual)
                e.res = p.residual[(int64_t)em * p.ldr + col];
            if (p.ln)
                e.wsum = p.w_rowsum[col];
        }
        return e;
    };

    int tile = blockIdx.x;
    // one column group ahead: with the weights on non-temporal loads a second group in flight no longer pays (measured on
    // the 768 -> 50257 shape: 28.5 us one ahead, 29.9 us two ahead, 32.9 us before either change)
    constexpr bool AHEAD2 = false;
    f32x4 w0[CHUNK], w1[CHUNK], w2[AHEAD2 ? CHUNK : 1];
    load_w(w0, tile);
    Epi e0 = load_epi(tile);
    Epi e1 { 0.f, 0.f, 0.f };
    if (AHEAD2 && tile + (int)gridDim.x < tiles) {
        load_w(w1, tile + gridDim.x);
        e1 = load_epi(tile + gridDim.x);
    }

    if (p.ln) { // statistics of the (at most 16) rows, from the registers that hold them; two-pass variance
        float s = 0.f;
#pragma unroll
        for (int c = 0; c < CHUNK; ++c)
            s += (a0[c][0] + a0[c][1]) + (a0[c][2] + a0[c][3]);
        s += __shfl_xor(s, 16, 64);
        s += __shfl_xor(s, 32, 64);
        if (kq == 0)
            stat[wave * 16 + i] = s;
        __syncthreads();
        if (t < 16) {
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w)
                tot += stat[w * 16 + t];
            row_mean[t] = tot / (float)K;
        }
        __syncthreads();
        const float mean = row_mean[i];
        float q = 0.f;
#pragma unroll
        for (int c = 0; c < CHUNK; ++c) {
            const int k = k_begin + c * 16 + kq * 4;
            if (c < slabs && k < k_end) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float d = a0[c][e] - mean;
                    q += d * d;
                }
            }
        }
        q += __shfl_xor(q, 16, 64);
        q += __shfl_xor(q, 32, 64);
        __syncthreads();
        if (kq == 0)
            stat[wave * 16 + i] = q;
        __syncthreads();
        if (t < 16) {
            float tot = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w)
                tot += stat[w * 16 + t];
            row_rstd[t] = 1.0f / sqrtf(tot / (float)K + p.ln_eps);
        }
        __syncthreads();
    }

    const int64_t len_shift = p.seg[0].len_stride ? (int64_t)(*p.len_dev) : 0; // only read when a segment asks for it
    unsigned long long best = 0ull; // packed maximum of this thread's output elements (one row, one column per group)
    int turn = 0;
    for (; tile < tiles; tile += gridDim.x) {
        float* red = red_both[turn];
        turn ^= 1;
        const int next = tile + (AHEAD2 ? 2 : 1) * gridDim.x;
        Epi e2 { 0.f, 0.f, 0.f };
        if (next < tiles) {
            if constexpr (AHEAD2)
                load_w(w2, next);
            else
                load_w(w1, next);
            e2 = load_epi(next);
        }
        f32x4 acc = { 0.f, 0.f, 0.f, 0.f };
#pragma unroll
        for (int s = 0; s < CHUNK; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a0[s][e], w0[s][e], acc, 0, 0, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            red[wave * 256 + (4 * kq + e) * 16 + i] = acc[e];
        __syncthreads();
        const int col = tile * 16 + ec;
        if (t < 256 && em < p.M && col < p.N) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < SK_WAVES; ++w)
                v += red[w * 256 + t];
            if (p.ln)
                v = row_rstd[em] * (v - row_mean[em] * e0.wsum);
            v = apply_act(v + e0.bias + e0.res, p.act);
            if (p.amax_parts) {
                const unsigned long long pk = pack_max(v, col);
                best = pk > best ? pk : best;
            }
            int sgi = 0;
            if (p.n_seg > 1 && col >= p.seg[1].col_begin)
                sgi = 1;
            if (p.n_seg > 2 && col >= p.seg[2].col_begin)
                sgi = 2;
            const SkinnySegment& sg = p.seg[sgi];
            const int64_t shift = sg.len_stride ? (sgi == 0 ? len_shift : (int64_t)(*p.len_dev)) * sg.len_stride : 0;
            sg.ptr[shift + (int64_t)em * sg.ld + (col - sg.col_begin)] = v;
        }
#pragma unroll
        for (int s = 0; s < CHUNK; ++s) {
            w0[s] = w1[s];
            if constexpr (AHEAD2)
                w1[s] = w2[s];
        }
        e0 = AHEAD2 ? e1 : e2;
        e1 = e2;
    }
    if (p.amax_parts && t < 256) { // the 16 lanes that share a row sit next to each other
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) {
            const unsigned long long other = __shfl_xor(best, o, 64);
            best = other > best ? other : best;
        }
        if (ec == 0)
            p.amax_parts[(int64_t)blockIdx.x * 16 + em] = best; // rows beyond M keep 0 = "no value"
    }
}

// [N][K] -> [column tile][wave][slab][lane] 16-byte pieces in exactly the order the GEMM's lanes consume
// them (lane l of wave w, slab s holds W[tile*16 + l%16][w*per_wave + s*16 + (l/16)*4 ..+3], zero beyond N or K),
// so every wave-wide load is one contiguous kilobyte
__global__ __launch_bounds__(64) void pack_weights_kernel(const float* __restrict__ w, int N, int K, int64_t ldw, int per_wave,
    float* __restrict__ out)
{
    const int spw = per_wave / 16;
    const int64_t blk = blockIdx.x; // ((tile * 8 + wave) * spw + slab)
    const int slab = (int)(blk % spw), wave = (int)((blk / spw) % SK_WAVES), tile = (int)(blk / ((int64_t)spw * SK_WAVES));
    const int lane = threadIdx.x;
    const int n = tile * 16 + (lane & 15), k = wave * per_wave + slab * 16 + (lane >> 4) * 4;
    f32x4 v = { 0.f, 0.f, 0.f, 0.f };
    if (n < N) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (k + e < K && k + e < (wave + 1) * per_wave)
                v[e] = w[(int64_t)n * ldw + k + e];
    }
    reinterpret_cast<f32x4*>(out)[blk * 64 + lane] = v;
}

// W'[n][k] = W[n][k] * gamma[k];  s[n] = sum_k W'[n][k];  b'[n] = b[n] + sum_k W[n][k] * beta[k]
__global__ __launch_bounds__(256) void fold_layernorm_kernel(const float* __restrict__ gamma, const float* __restrict__ beta,
    const float* __restrict__ w, const float* __restrict__ bias, int k, float* __restrict__ w_out, float* __restrict__ wsum,
    float* __restrict__ bias_out)
{
    __shared__ float sa[4], sb[4];
    const int n = blockIdx.x;
    const float* wr = w + (int64_t)n * k;
    float* wo = w_out + (int64_t)n * k;
    float s = 0.f, bsum = 0.f;
    for (int z = threadIdx.x; z < k; z += 256) {
        const float wv = wr[z];
        const float folded = wv * (gamma ? gamma[z] : 1.f);
        wo[z] = folded;
        s += folded;
        bsum += wv * (beta ? beta[z] : 0.f);
    }
    for (int o = 32; o > 0; o >>= 1) {
        s += __shfl_xor(s, o, 64);
        bsum += __shfl_xor(bsum, o, 64);
    }
    if ((threadIdx.x & 63) == 0) {
        sa[threadIdx.x >> 6] = s;
        sb[threadIdx.x >> 6] = bsum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        wsum[n] = (sa[0] + sa[1]) + (sa[2] + sa[3]);
        bias_out[n] = (bias ? bias[n] : 0.f) + ((sb[0] + sb[1]) + (sb[2] + sb[3]));
    }
}

// out[b][:] = table_a[ids[b]][:] + table_b[*len_dev][:]  (token + position embedding of one new token);
// also clears this sequence's packed arg-max cell for the step's last kernel
__global__ void embed_add_kernel(const float* __restrict__ ids, const float* __restrict__ ta, int dim_a,
    const float* __restrict__ tb, int dim_b, const int* __restrict__ len_dev, int depth, float* __restrict__ out,
    int* __restrict__ err, unsigned long long* __restrict__ amax)
{
    const int b = blockIdx.x;
    const float f = ids[b];
    int64_t id = (f >= 0.f && f < 9.0e18f) ? (int64_t)f : -1;
    const int64_t pos = *len_dev;
    const bool ok = id >= 0 && id < dim_a && pos < dim_b;
    if (!ok && err && threadIdx.x == 0)
        atomicExch(err, 1);
    if (amax && threadIdx.x == 0)
        amax[b] = 0ull;
    for (int z = threadIdx.x; z < depth; z += blockDim.x)
        out[(int64_t)b * depth + z] = ok ? ta[id * depth + z] + tb[pos * depth + z] : 0.f;
}

// One workgroup per (sequence, head); the number of visible keys is *len_dev + 1 (the new token's
// key / value row was written by the projection kernel just before).
__global__ __launch_bounds__(256) void mha_decode_dyn_kernel(const float* __restrict__ q, int64_t ldq,
    const float* __restrict__ kc, const float* __restrict__ vc, float* __restrict__ out, int heads, int dk, int dv,
    const int* __restrict__ len_dev, int max_len, float scale)
{
    extern __shared__ float smem[]; // [dk] query, [max_len] scores, [256] reduction scratch
    const int len = *len_dev + 1;
    float* sq = smem;
    float* sp = smem + dk;
    float* red = sp + max_len;
    const int b = blockIdx.x / heads, h = blockIdx.x % heads, tid = threadIdx.x;
    const int64_t krow = (int64_t)heads * dk, vrow = (int64_t)heads * dv;
    for (int d = tid; d < dk; d += 256)
        sq[d] = q[(int64_t)b * ldq + h * dk + d];
    __syncthreads();
    // scores: 16 lanes share one key row (each lane 16 contiguous bytes per pass), so a wave reads four
    // whole rows per load; four passes are issued together to keep more rows in flight
    float m = -FLT_MAX;
    const int part = tid & 15, slot = tid >> 4;
    const float* kbase = kc + (int64_t)b * max_len * krow + h * dk;
    if (dk == 64) {
        const f32x4 qv = *reinterpret_cast<const f32x4*>(sq + part * 4);
        for (int j0 = 0; j0 < len; j0 += 64) {
            f32x4 kv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = j0 + u * 16 + slot;
                kv[u] = f32x4 { 0.f, 0.f, 0.f, 0.f };
                if (j < len)
                    kv[u] = *reinterpret_cast<const f32x4*>(kbase + (int64_t)j * krow + part * 4);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = j0 + u * 16 + slot;
                float s = qv[0] * kv[u][0] + qv[1] * kv[u][1] + qv[2] * kv[u][2] + qv[3] * kv[u][3];
                for (int o = 8; o > 0; o >>= 1)
                    s += __shfl_xor(s, o, 64);
                if (j < len) {
                    s *= scale;
                    if (part == 0)
                        sp[j] = s;
                    m = fmaxf(m, s);
                }
            }
        }
    } else {
        for (int j0 = 0; j0 < len; j0 += 16) {
            const int j = j0 + slot;
            float s = 0.f;
            if (j < len)
                for (int d = part; d < dk; d += 16)
                    s += sq[d] * kbase[(int64_t)j * krow + d];
            for (int o = 8; o > 0; o >>= 1)
                s += __shfl_xor(s, o, 64);
            if (j < len) {
                s *= scale;
                if (part == 0)
                    sp[j] = s;
                m = fmaxf(m, s);
            }
        }
    }
    __syncthreads();
    for (int o = 32; o > 0; o >>= 1)
        m = fmaxf(m, __shfl_xor(m, o, 64));
    if ((tid & 63) == 0)
        red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    float sum = 0.f;
    for (int j = tid; j < len; j += 256)
        sum += expf(sp[j] - m);
    for (int o = 32; o > 0; o >>= 1)
        sum += __shfl_xor(sum, o, 64);
    __syncthreads();
    if ((tid & 63) == 0)
        red[tid >> 6] = sum;
    __syncthreads();
    const float ls = logf(red[0] + red[1] + red[2] + red[3]);
    for (int j = tid; j < len; j += 256) {
        const float pr = expf(sp[j] - m - ls);
        sp[j] = isinf(pr) ? 0.f : pr;
    }
    __syncthreads();
    // P V: lanes along the value depth, 256/dv key partitions; eight rows in flight per thread
    const int parts = dv <= 256 ? 256 / dv : 1;
    const float* vbase = vc + (int64_t)b * max_len * vrow + h * dv;
    for (int d0 = 0; d0 < dv; d0 += 256) {
        const int d = d0 + (parts > 1 ? tid % dv : tid), prt = parts > 1 ? tid / dv : 0;
        float acc = 0.f;
        if (d < dv && prt < parts) {
            for (int j0 = prt; j0 < len; j0 += 8 * parts) {
                float vv[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int j = j0 + u * parts;
                    vv[u] = j < len ? vbase[(int64_t)j * vrow + d] : 0.f;
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int j = j0 + u * parts;
                    if (j < len)
                        acc += sp[j] * vv[u];
                }
            }
        }
        if (parts > 1) {
            __syncthreads();
            red[tid] = acc;
            __syncthreads();
            if (tid < dv) {
                float r = red[tid];
                for (int pidx = 1; pidx < parts; ++pidx)
                    r += red[pidx * dv + tid];
                out[(int64_t)b * vrow + h * dv + tid] = r;
            }
        } else if (d < dv) {
            out[(int64_t)b * vrow + h * dv + d] = acc;
        }
    }
}

// Packs (value, column) so that an unsigned 64-bit max picks the largest value and, among equal values,
// the smallest column: the first maximum wins, as in the reference's tensor_max_pos.
__device__ __forceinline__ unsigned long long pack_max(float v, int col)
{
    unsigned int u = __float_as_uint(v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u); // order-preserving map of floats to unsigned
    return ((unsigned long long)u << 32) | (unsigned long long)(0xFFFFFFFFu - (unsigned int)col);
}

// per-row partial arg-max over a slice of columns, merged with a 64-bit atomic max
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ x, int depth, int cols_per_block,
    unsigned long long* __restrict__ amax)
{
    __shared__ unsigned long long sm[4];
    const int row = blockIdx.y, c0 = blockIdx.x * cols_per_block;
    const int c1 = c0 + cols_per_block < depth ? c0 + cols_per_block : depth;
    const float* xr = x + (int64_t)row * depth;
    unsigned long long best = 0ull;
    for (int z = c0 + threadIdx.x; z < c1; z += 256) {
        const unsigned long long pk = pack_max(xr[z], z);
        best = pk > best ? pk : best;
    }
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(best, o, 64);
        best = other > best ? other : best;
    }
    if ((threadIdx.x & 63) == 0)
        sm[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            best = sm[w] > best ? sm[w] : best;
        atomicMax(&amax[row], best);
    }
}

// per-workgroup partial maxima [parts][16] -> float ids, then as argmax_finish_kernel
__global__ __launch_bounds__(1024) void argmax_parts_kernel(const unsigned long long* __restrict__ parts, int n_parts, int rows,
    float* __restrict__ out_idx_f, int* __restrict__ len_dev, float* __restrict__ history)
{
    __shared__ unsigned long long sm[64][16];
    const int r = threadIdx.x & 15, lane_part = threadIdx.x >> 4; // 64 threads per row
    unsigned long long best = 0ull;
    for (int q = lane_part; q < n_parts; q += 64) {
        const unsigned long long pk = parts[(int64_t)q * 16 + r];
        best = pk > best ? pk : best;
    }
    sm[lane_part][r] = best;
    __syncthreads();
    if (threadIdx.x < 16 && r < rows) {
        for (int q = 0; q < 64; ++q)
            best = sm[q][r] > best ? sm[q][r] : best;
        const float id = best == 0ull ? 0.f : (float)(0xFFFFFFFFu - (unsigned int)(best & 0xFFFFFFFFull));
        out_idx_f[r] = id;
        if (history && len_dev)
            history[(int64_t)(*len_dev) * rows + r] = id;
    }
    __syncthreads();
    if (len_dev && threadIdx.x == 0)
        *len_dev += 1;
}

// The same, and the embedding of the tokens just picked at the position they will take, x0[r][:] = table_a[id_r][:] +
// table_b[new length][:]: inside a greedy loop this is the first launch of the next step (embed_add_kernel) riding in the
// last launch of this one.  Ids beyond table_a cannot occur (they are column numbers of the head); a position beyond
// table_b leaves zeros and reports nothing: the loop's last step embeds for a step that may never come (the caller keeps
// loops that would run past the table on the stand-alone launch).
__global__ __launch_bounds__(1024) void argmax_parts_embed_kernel(const unsigned long long* __restrict__ parts, int n_parts, int rows,
    float* __restrict__ out_idx_f, int* __restrict__ len_dev, float* __restrict__ history, const float* __restrict__ ta, int dim_a,
    const float* __restrict__ tb, int dim_b, int depth, float* __restrict__ x0, int* __restrict__ err)
{
    __shared__ unsigned long long sm[64][16];
    __shared__ int ids_s[16];
    __shared__ int pos_s;
    const int r = threadIdx.x & 15, lane_part = threadIdx.x >> 4; // 64 threads per row
    unsigned long long best = 0ull;
    for (int q = lane_part; q < n_parts; q += 64) {
        const unsigned long long pk = parts[(int64_t)q * 16 + r];
        best = pk > best ? pk : best;
    }
    sm[lane_part][r] = best;
    __syncthreads();
    if (threadIdx.x < 16 && r < rows) {
        for (int q = 0; q < 64; ++q)
            best = sm[q][r] > best ? sm[q][r] : best;
        const unsigned int col = best == 0ull ? 0u : 0xFFFFFFFFu - (unsigned int)(best & 0xFFFFFFFFull);
        const float id = (float)col;
        out_idx_f[r] = id;
        history[(int64_t)(*len_dev) * rows + r] = id;
        ids_s[r] = (int)col;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int pos = *len_dev + 1;
        *len_dev = pos;
        pos_s = pos;
    }
    __syncthreads();
    const int pos = pos_s, quads = depth / 4;
    for (int idx = threadIdx.x; idx < rows * quads; idx += 1024) {
        const int row = idx / quads, c4 = (idx - row * quads) * 4;
        const int id = ids_s[row];
        f32x4 v = { 0.f, 0.f, 0.f, 0.f };
        if (id < dim_a && pos < dim_b)
            v = *reinterpret_cast<const f32x4*>(ta + (int64_t)id * depth + c4) + *reinterpret_cast<const f32x4*>(tb + (int64_t)pos * depth + c4);
        *reinterpret_cast<f32x4*>(x0 + (int64_t)row * depth + c4) = v;
    }
}

// packed winners -> float ids; optionally advances the session length (every other kernel of the step
// has finished by stream order)
__global__ void argmax_finish_kernel(const unsigned long long* __restrict__ amax, int rows, float* __restrict__ out_idx_f,
    int* __restrict__ len_dev, float* __restrict__ history)
{
    const int r = threadIdx.x;
    if (r < rows) {
        const unsigned long long pk = amax[r];
        const float id = pk == 0ull ? 0.f : (float)(0xFFFFFFFFu - (unsigned int)(pk & 0xFFFFFFFFull));
        out_idx_f[r] = id;
        if (history && len_dev)
            history[(int64_t)(*len_dev) * rows + r] = id; // row = position of the token that produced these logits
    }
    __syncthreads();
    if (len_dev && r == 0)
        *len_dev += 1;
}

__global__ void set_int_kernel(int* p, int v) { *p = v; }

// library-owned scratch of the split-K path: partial tiles and one ticket per column tile (zero between launches)
constexpr int64_t kSplitWsFloats = 1 << 20;
constexpr int kSplitTickets = 4096;
static float* g_splitk_ws = nullptr;
static int* g_splitk_tickets = nullptr;
static bool ensure_splitk_workspace()
{
    if (g_splitk_ws && g_splitk_tickets)
        return true;
    if (hipMalloc(&g_splitk_ws, sizeof(float) * kSplitWsFloats) != hipSuccess)
        return false;
    if (hipMalloc(&g_splitk_tickets, sizeof(int) * kSplitTickets) != hipSuccess
        || zero_device(g_splitk_tickets, sizeof(int) * kSplitTickets) != hipSuccess)
        return false;
    return true;
}

// workgroups of the wide-output kernel that are resident at once (queried once, outside any stream capture)
static int wide_resident()
{
    static const int resident = [] {
        int per_cu = 1, dev = 0, cus = 256;
        hipDeviceProp_t prop;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, skinny_wide_kernel<SK_CHUNK>, 512, 0) != hipSuccess || per_cu < 1)
            per_cu = 1;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            cus = prop.multiProcessorCount;
        return per_cu * cus;
    }();
    return resident;
}

// allocates the split-K scratch ahead of time (it must not happen inside a stream capture)
fdx_status skinny_prepare()
{
    (void)wide_resident();
    if (!ensure_splitk_workspace()) {
        set_error("dense_rows: out of device memory for the split-K workspace");
        return FDX_ERR_HIP;
    }
    return FDX_OK;
}

// (rows this short are never split along K, so the choice depends on K and the number of column groups alone)
int skinny_wide_grid(const SkinnyParams& p)
{
    const int tiles = (p.N + 15) / 16;
    if (p.M <= 0 || p.M > 16 || p.K <= 0)
        return 0;
    const int per_wg = ((p.K + 15) / 16) * 16;
    const int grid = wide_resident();
    return (per_wg <= SK_WAVES * SK_CHUNK * 16 && tiles >= 4 * grid) ? grid : 0;
}

fdx_status argmax_parts_launch(const unsigned long long* amax_parts, int parts, int rows, float* out_idx_f, int* len_dev, float* history)
{
    FDX_REQUIRE(amax_parts && out_idx_f && parts > 0 && rows > 0 && rows <= 16, "argmax: bad arguments");
    profile_begin();
    hipLaunchKernelGGL(argmax_parts_kernel, dim3(1), dim3(1024), 0, stream(), amax_parts, parts, rows, out_idx_f, len_dev, history);
    profile_end("argmax_f32", 0.0, 8.0 * parts * 16);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

fdx_status argmax_parts_embed_launch(const unsigned long long* amax_parts, int parts, int rows, float* out_idx_f, int* len_dev, float* history,
    const float* ta, int dim_a, const float* tb, int dim_b, int depth, float* x0, int* err)
{
    FDX_REQUIRE(amax_parts && out_idx_f && len_dev && history && ta && tb && x0 && parts > 0 && rows > 0 && rows <= 16 && depth > 0
            && depth % 4 == 0 && (reinterpret_cast<uintptr_t>(ta) & 15) == 0 && (reinterpret_cast<uintptr_t>(tb) & 15) == 0
            && (reinterpret_cast<uintptr_t>(x0) & 15) == 0,
        "argmax_embed: bad arguments");
    profile_begin();
    hipLaunchKernelGGL(argmax_parts_embed_kernel, dim3(1), dim3(1024), 0, stream(), amax_parts, parts, rows, out_idx_f, len_dev, history, ta,
        dim_a, tb, dim_b, depth, x0, err);
    profile_end("argmax_f32", 0.0, 8.0 * parts * 16 + 12.0 * rows * depth);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

// K ranges per column group of a launch without LayerNorm prologue and pre-packed operand
static int skinny_ksplit(int K, int tiles)
{
    // spread a narrow projection over the chip: a CU pulls only a few tens of GB/s on its own
    // long K only: below that the ticket exchange costs more than the idle CUs
    int ksplit = 1;
    while (ksplit < 8 && K / ksplit > SK_WAVES * SK_CHUNK * 16 && K / (ksplit * 2) >= 128)
        ksplit *= 2;
    if (ksplit > 1)
        while (ksplit < 8 && tiles * ksplit < 192 && K / (ksplit * 2) >= 256)
            ksplit *= 2;
    return ksplit;
}

fdx_status skinny_gemm_launch(const SkinnyParams& p)
{
    FDX_REQUIRE((p.X || p.emb_x) && p.W && p.M > 0 && p.M <= 16 && p.N > 0 && p.K > 0, "dense_rows: bad arguments");
    FDX_REQUIRE(!(p.emb_x || p.emb_res) || (p.emb_ids && p.emb_a && p.emb_b && p.len_dev && p.emb_a_rows > 0 && p.emb_b_rows > 0),
        "dense_rows: the embedding prologue needs ids, both tables and the position counter");
    FDX_REQUIRE(p.K % 4 == 0 && p.ldx % 4 == 0 && p.ldw % 4 == 0, "dense_rows: K and row strides must be multiples of 4");
    FDX_REQUIRE(p.n_seg >= 1 && p.n_seg <= 3, "dense_rows: 1 to 3 output segments");
    FDX_REQUIRE(!p.ln || (p.K <= SK_WAVES * SK_CHUNK * 16 && p.w_rowsum), "dense_rows: the LayerNorm prologue needs K <= %d",
        SK_WAVES * SK_CHUNK * 16);
    FDX_REQUIRE(!p.residual || p.residual != p.seg[0].ptr, "dense_rows: the residual is read before the output is written; they must not alias");
    const int tiles = (p.N + 15) / 16;
    // split K across workgroups when a launch would otherwise leave most CUs idle or a wave would need
    // more than one chunk; LayerNorm launches keep whole rows in one workgroup
    int ksplit = 1;
    SkinnyParams q = p;
    // the caller's workspace (the entry point that allocates nothing brings its own) or the library's, allocated on first use
    const bool own_ws = p.workspace && p.tickets;
    if (!p.ln && !p.packed && (own_ws || ensure_splitk_workspace())) {
        const int64_t ws_floats = own_ws ? p.workspace_floats : kSplitWsFloats;
        const int ticket_count = own_ws ? p.ticket_count : kSplitTickets;
        ksplit = skinny_ksplit(p.K, tiles);
        if ((int64_t)tiles * ksplit * 256 > ws_floats || tiles > ticket_count)
            ksplit = 1;
        if (!own_ws) {
            q.workspace = g_splitk_ws;
            q.tickets = g_splitk_tickets;
        }
        // column groups in a multiple of 8: the K ranges of a group share an XCD and meet in its L2 (FDX_SPLIT_LOCAL=0
        // keeps the exchange through memory, for comparison)
        static const bool local_on = [] { const char* e = std::getenv("FDX_SPLIT_LOCAL"); return !(e && e[0] == '0'); }();
        q.ticket_count = ticket_count;
        q.workspace_floats = ws_floats;
        q.local_split = (int)(local_on && ksplit > 1 && ksplit <= 8 && tiles % 8 == 0 && tiles * 8 <= ticket_count / 2 && tiles <= ticket_count / 2);
        q.err = async_error_cell();
    }
    const int per_wg = ((p.K + ksplit * 16 - 1) / (ksplit * 16)) * 16; // as the kernel derives it
    const dim3 grid((unsigned)tiles, (unsigned)ksplit);
    profile_begin();
    // many column groups and a short K: resident workgroups stride through the groups instead of one group each
    const int wide_grid = skinny_wide_grid(p);
    FDX_REQUIRE(!p.amax_parts || (wide_grid > 0 && ksplit == 1), "dense_rows: partial arg-max cells need the wide-output kernel");
    FDX_REQUIRE(!(p.emb_x || p.emb_res) || (wide_grid == 0 && ksplit == 1 && per_wg <= SK_WAVES * 6 * 16),
        "dense_rows: the embedding prologue needs K <= %d and runs neither with the wide-output kernel nor with K split across workgroups",
        SK_WAVES * 6 * 16);
    if (ksplit == 1 && wide_grid > 0) {
        if (per_wg <= SK_WAVES * 6 * 16)
            hipLaunchKernelGGL((skinny_wide_kernel<6>), dim3((unsigned)wide_grid), dim3(512), 0, stream(), q, tiles);
        else
            hipLaunchKernelGGL((skinny_wide_kernel<SK_CHUNK>), dim3((unsigned)wide_grid), dim3(512), 0, stream(), q, tiles);
        profile_end("dense_rows_f32", 2.0 * p.M * (double)p.N * p.K, 4.0 * ((double)p.N * p.K + (double)p.M * (p.K + p.N)));
        FDX_LAUNCH_CHECK();
        return FDX_OK;
    }
    // every load of a workgroup in flight at once when its K range fits 8 (or 24) slabs per wave
    if (p.emb_x || p.emb_res)
        hipLaunchKernelGGL((skinny_gemm_kernel<6, true, true>), grid, dim3(512), 0, stream(), q);
    else if (per_wg <= SK_WAVES * 6 * 16) // K = 768 and the halves / quarters of longer rows: no empty register slots
        hipLaunchKernelGGL((skinny_gemm_kernel<6, true>), grid, dim3(512), 0, stream(), q);
    else if (per_wg <= SK_WAVES * SK_CHUNK * 16)
        hipLaunchKernelGGL((skinny_gemm_kernel<SK_CHUNK, true>), grid, dim3(512), 0, stream(), q);
    else if (per_wg <= SK_WAVES * SK_CHUNK_LONG * 16)
        hipLaunchKernelGGL((skinny_gemm_kernel<SK_CHUNK_LONG, true>), grid, dim3(512), 0, stream(), q);
    else
        hipLaunchKernelGGL((skinny_gemm_kernel<SK_CHUNK, false>), grid, dim3(512), 0, stream(), q);
    profile_end("dense_rows_f32", 2.0 * p.M * (double)p.N * p.K, 4.0 * ((double)p.N * p.K + (double)p.M * (p.K + p.N)));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

// number of floats pack_weights_launch writes for an [n][k] operand
int64_t packed_weight_floats(int n, int k)
{
    const int per_wave = ((k + SK_WAVES * 16 - 1) / (SK_WAVES * 16)) * 16;
    return (int64_t)((n + 15) / 16) * SK_WAVES * (per_wave / 16) * 64 * 4;
}

fdx_status pack_weights_launch(const float* w, int n, int k, int64_t ldw, float* out)
{
    FDX_REQUIRE(w && out && n > 0 && k > 0, "pack_weights: bad arguments");
    const int per_wave = ((k + SK_WAVES * 16 - 1) / (SK_WAVES * 16)) * 16;
    const int64_t blocks = (int64_t)((n + 15) / 16) * SK_WAVES * (per_wave / 16);
    hipLaunchKernelGGL(pack_weights_kernel, dim3((unsigned)blocks), dim3(64), 0, stream(), w, n, k, ldw, per_wave, out);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

fdx_status fold_layernorm_launch(const float* gamma, const float* beta, const float* w, const float* bias, int n, int k,
    float* w_out, float* wsum, float* bias_out)
{
    FDX_REQUIRE(w && w_out && wsum && bias_out && n > 0 && k > 0, "fold_layernorm: bad arguments");
    hipLaunchKernelGGL(fold_layernorm_kernel, dim3((unsigned)n), dim3(256), 0, stream(), gamma, beta, w, bias, k, w_out, wsum, bias_out);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

fdx_status embed_add_launch(const float* ids, int batch, const float* ta, int dim_a, const float* tb, int dim_b,
    const int* len_dev, int depth, float* out, int* err, unsigned long long* amax)
{
    FDX_REQUIRE(ids && ta && tb && len_dev && out && batch > 0 && depth > 0, "embed_add: bad arguments");
    profile_begin();
    hipLaunchKernelGGL(embed_add_kernel, dim3(batch), dim3(256), 0, stream(), ids, ta, dim_a, tb, dim_b, len_dev, depth, out, err, amax);
    profile_end("embed_add_f32", 0.0, 12.0 * batch * depth);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

bool mha_decode_fast_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch, int heads,
    int dk, int dv, const int* len_dev, int max_len, hipStream_t s);

fdx_status mha_decode_dyn_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch,
    int heads, int dk, int dv, const int* len_dev, int max_len, int len_hint)
{
    FDX_REQUIRE(q && kc && vc && out && len_dev && batch > 0 && heads > 0 && dk > 0 && dv > 0 && max_len > 0, "mha_decode: bad arguments");
    const size_t smem = sizeof(float) * ((size_t)dk + max_len + 256);
    FDX_REQUIRE(smem <= 64 * 1024, "mha_decode: max_len %d exceeds the single-pass kernel's LDS budget", max_len);
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    profile_begin();
    if (!mha_decode_fast_launch(q, ldq, kc, vc, out, batch, heads, dk, dv, len_dev, max_len, stream()))
        hipLaunchKernelGGL(mha_decode_dyn_kernel, dim3(batch * heads), dim3(256), smem, stream(), q, ldq, kc, vc, out, heads, dk, dv,
            len_dev, max_len, scale);
    profile_end("mha_decode_f32", 4.0 * batch * heads * (double)len_hint * dk, 4.0 * (double)batch * len_hint * heads * (dk + dv));
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

// amax must hold zeros on entry (embed_add_kernel clears it at the start of every step)
fdx_status argmax_bump_launch(const float* x, int rows, int depth, float* out_idx_f, int* len_dev, unsigned long long* amax,
    float* history)
{
    FDX_REQUIRE(x && out_idx_f && amax && rows > 0 && rows <= 1024 && depth > 0, "argmax: bad arguments");
    const int cols_per_block = 2048;
    profile_begin();
    hipLaunchKernelGGL(argmax_partial_kernel, dim3((unsigned)((depth + cols_per_block - 1) / cols_per_block), (unsigned)rows), dim3(256), 0,
        stream(), x, depth, cols_per_block, amax);
    hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(1024), 0, stream(), amax, rows, out_idx_f, len_dev, history);
    profile_end("argmax_f32", 0.0, 4.0 * rows * depth);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

fdx_status set_int_launch(int* p, int v)
{
    hipLaunchKernelGGL(set_int_kernel, dim3(1), dim3(1), 0, stream(), p, v);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

} // namespace fdx

// ---- C ABI (include/fdx.h documents the semantics)
extern "C" fdx_status fdx_dense_rows_f32(const float* x, int m, int k, const float* w_nk, const float* bias, int n,
    const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(x && w_nk && out, "dense_rows: null pointer");
    fdx::SkinnyParams p;
    std::memset(&p, 0, sizeof p);
    p.X = x; p.ldx = k; p.W = w_nk; p.ldw = k; p.M = m; p.N = n; p.K = k; p.bias = bias; p.residual = residual; p.ldr = n;
    FDX_REQUIRE_EPILOGUE_ACT(act);
    p.act = fdx::make_act(act);
    p.n_seg = 1;
    p.seg[0] = { out, n, 0, 0 };
    return fdx::skinny_gemm_launch(p);
}

// ---- the Dense entry point that allocates nothing -----------------------------------------------------------------
// Split-K partial tiles and tickets of fdx_dense_rows_noalloc_f32 live in this file-scope device array instead of
// memory from hipMalloc: [kNoAllocWsFloats] partial-tile floats, then [kNoAllocTickets] ticket ints.  The GPU holds
// it (4 MiB + 16 KiB) until the process ends.  Host code never passes the array's name to a kernel: its device
// address is looked up once, at library set-up, and kept in g_noalloc_ptr.
namespace fdx {
constexpr int64_t kNoAllocWsFloats = 1 << 20;
constexpr int kNoAllocTickets = 4096;
static __device__ __align__(256) float scratch[kNoAllocWsFloats + kNoAllocTickets];
static float* g_noalloc_ptr = nullptr; // device address of `scratch` on the library's device

__global__ void clear_ints_kernel(int* p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        p[i] = 0;
}

// called from the library's set-up (runtime.cpp:ensure_init) with the library's device current
hipError_t noalloc_setup()
{
    (void)wide_resident(); // occupancy query of the wide-output kernel, cached: not to be made inside a capture
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess)
        return e;
    g_noalloc_ptr = static_cast<float*>(ptr);
    return hipSuccess;
}
} // namespace fdx

extern "C" fdx_status fdx_dense_rows_noalloc_f32(const float* x, int m, int k, const float* w_nk, const float* bias, int n,
    const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(x && w_nk && out, "dense_rows_noalloc: null pointer");
    FDX_REQUIRE(fdx::g_noalloc_ptr, "dense_rows_noalloc: call fdx_init first (the library's set-up looks up the scratch array's address)");
    FDX_REQUIRE(m > 0 && m <= 16, "dense_rows_noalloc: 1 to 16 rows, got %d", m);
    FDX_REQUIRE(n > 0 && n <= 16 * fdx::kNoAllocTickets, "dense_rows_noalloc: at most %d output columns, got %d", 16 * fdx::kNoAllocTickets, n);
    FDX_REQUIRE(k > 0 && k <= 32768, "dense_rows_noalloc: at most 32768 input columns, got %d", k);
    const int tiles = (n + 15) / 16;
    const int ksplit = fdx::skinny_ksplit(k, tiles);
    FDX_REQUIRE((int64_t)tiles * ksplit * 256 <= fdx::kNoAllocWsFloats,
        "dense_rows_noalloc: %d column groups x %d K ranges exceed the fixed scratch of %lld floats", tiles, ksplit,
        (long long)fdx::kNoAllocWsFloats);
    fdx::SkinnyParams p;
    std::memset(&p, 0, sizeof p);
    p.X = x; p.ldx = k; p.W = w_nk; p.ldw = k; p.M = m; p.N = n; p.K = k; p.bias = bias; p.residual = residual; p.ldr = n;
    FDX_REQUIRE_EPILOGUE_ACT(act);
    p.act = fdx::make_act(act);
    p.n_seg = 1;
    p.seg[0] = { out, n, 0, 0 };
    p.workspace = fdx::g_noalloc_ptr;
    p.workspace_floats = fdx::kNoAllocWsFloats;
    p.tickets = reinterpret_cast<int*>(fdx::g_noalloc_ptr + fdx::kNoAllocWsFloats);
    p.ticket_count = fdx::kNoAllocTickets;
    if (ksplit > 1) {
        // every call on this GPU shares the array, which keeps the last call's contents: the tickets this launch counts
        // on start at zero (a fill kernel, not a memset, so that a caller may capture the call)
        hipLaunchKernelGGL(fdx::clear_ints_kernel, dim3((unsigned)((tiles + 255) / 256)), dim3(256), 0, fdx::stream(), p.tickets, tiles);
        FDX_LAUNCH_CHECK();
    }
    return fdx::skinny_gemm_launch(p);
}

extern "C" fdx_status fdx_fold_layernorm_f32(const float* gamma, const float* beta, const float* w_nk, const float* bias, int n,
    int k, float* w_folded, float* w_rowsum, float* bias_folded)
{
    return fdx::fold_layernorm_launch(gamma, beta, w_nk, bias, n, k, w_folded, w_rowsum, bias_folded);
}

extern "C" fdx_status fdx_layernorm_dense_rows_f32(const float* x, int m, int k, float ln_eps, const float* w_folded,
    const float* w_rowsum, const float* bias_folded, int n, const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(x && w_folded && w_rowsum && out, "layernorm_dense_rows: null pointer");
    fdx::SkinnyParams p;
    std::memset(&p, 0, sizeof p);
    p.X = x; p.ldx = k; p.W = w_folded; p.ldw = k; p.M = m; p.N = n; p.K = k; p.bias = bias_folded; p.residual = residual; p.ldr = n;
    FDX_REQUIRE_EPILOGUE_ACT(act);
    p.act = fdx::make_act(act);
    p.ln = 1; p.ln_eps = ln_eps; p.w_rowsum = w_rowsum;
    p.n_seg = 1;
    p.seg[0] = { out, n, 0, 0 };
    return fdx::skinny_gemm_launch(p);
}

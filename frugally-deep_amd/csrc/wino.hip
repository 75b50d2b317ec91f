// 3x3 stride-1 convolution in the Winograd F(2x2, 3x3) form on fp32 MFMA, gfx950.
//
// A 3x3 convolution spends 9 multiply-adds per output pixel and channel pair.  Computed on 2x2 output tiles from their
// 4x4 input patches d with the filter g moved into the same 4x4 domain once at load,
//     Y = At [ sum_c (G g_c Gt) o (Bt d_c B) ] A          (o = element by element),
// it spends 16 per four pixels, 2.25 times fewer: for each of the 16 positions of the 4x4 domain the sum over the input
// channels is a GEMM  M_p[tile][cout] = sum_c V_p[tile][c] * U_p[c][cout],  and those run on the matrix cores.
//
// A unit of work is 32 tiles (of any images, in raster order) by NT * 32 output channels; a workgroup of four waves
// works on one unit at a time (how units are dealt to workgroups: see wino_kernel).  Wave xi owns
// row xi of the 4x4 domain, i.e. the four positions (xi, 0..3):
//   * per step of 8 input channels a lane takes, for its tile (lane % 32) and its four channels (lane / 32), the two
//     patch rows that row xi of Bt combines, four pixels each, straight from global memory (a pixel outside the image
//     is an out-of-range buffer offset and reads as zero: the convolution's padding), forms the four transformed
//     values with 8 additions per channel, and has the A operands of its four GEMMs in registers -- no LDS, no barrier;
//   * the B operands come from the transformed filter, laid out at load so that what a wave takes for one position,
//     one column tile and one step is one contiguous kilobyte: U[cout / 32][cin / 8][position][lane][4], lane =
//     32 * (channel / 4 % 2) + cout % 32;
//   * 4 positions x NT column tiles of 32x32x2 MFMA accumulate over the input channels.
// At the end each wave folds its four positions with At along the row (two values per tile and channel), the four
// waves meet once in LDS, and wave (i, j) combines the rows with At along the column into output pixel (i, j) of
// every tile, adds bias and residual, applies the activation and stores 16-byte pieces.
//
// Transform matrices (Lavin & Gray, "Fast Algorithms for Convolutional Neural Networks", F(2x2, 3x3)):
//   Bt = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]   G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1]   At = [1 1 1 0; 0 1 -1 -1]
// Their entries are 0, +-1 and +-1/2: the result differs from the direct sum by a few more roundings (measured against
// the reference's order of summation in the tests), not by a conditioning problem as the larger tiles have.
//
// Replaces convolve for 3x3 filters, stride 1, no dilation (include/fdeep/convolution.hpp:398-429, :107-160).
#include <cstring>
#include <mutex>

#include "common.hpp"
#include "igemm_params.hpp"

namespace fdx {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

struct WinoParams {
    const float* in;       // [n][h][w][cin]
    const float* u;        // [cout / 32][cin / 8][16][64][4], see fdx_conv2d_winograd_prepare
    const float* bias;     // [cout] or null
    const float* residual; // like out, or null
    float* out;            // [n][oh][ow][cout]
    int n, h, w, cin, cout, pad_top, pad_left, oh, ow;
    int tiles_x, tiles_y, tiles; // 2x2 output tiles per row, per image column, and all of them
    uint32_t in_bytes, out_bytes, u_bytes, ws_bytes;
    int m_blocks, n_blocks, units; // blocks of 32 tiles, column blocks of NT * 32 channels; units of work = their product
    int nb_group;        // column blocks per group: units are ordered group, tile block, column block inside the group
    int per_wg, longer;  // steps per workgroup (total / workgroups) and how many workgroups take one more
    float* ws;           // shares of units that several workgroups work on: two places per workgroup
    int* tickets;        // one per unit, zero between launches
    Act act;
};

constexpr int WINO_TM = 32;  // tiles per workgroup
constexpr int WINO_PAD = 4;  // padding of an LDS row of the exchange

// one step's operands: the eight patch pixels of this lane's tile and the 4 x NT filter pieces of its positions
template <int NT>
__device__ __forceinline__ void wino_load(f32x4 (&dd)[2][4], f32x4 (&bb)[4][NT], const uint32_t (&pix_off)[2][4],
    const uint32_t (&u_off)[4][NT], const __amdgpu_buffer_rsrc_t& srd_in, const __amdgpu_buffer_rsrc_t& srd_u, int step)
{
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < 4; ++j)
            dd[r][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_in, (int)pix_off[r][j], step * 32, 0));
#pragma unroll
    for (int nu = 0; nu < 4; ++nu)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            bb[nu][nt] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_u, (int)u_off[nu][nt], step * 16384, 0));
}

// One step: 8 input channels into the 4 x NT accumulators of this wave.  There is one register set of operands, and
// with AHEAD each register is asked for its next step's value as soon as this step has read it -- the patch pixels right
// after the input transform, the filter pieces of a position right after its MFMAs -- so that every load has a whole
// step to arrive in while the registers of a second set stay free: at 128 accumulators + 64 operand registers two
// workgroups fit on a CU, and the end of one's unit (exchange, barriers, stores) runs under the other's MFMAs.
// NT = 32-column tiles of the output channels per workgroup, XI = this wave's row of the transform domain.
template <int NT, int XI, bool AHEAD>
__device__ __forceinline__ void wino_step(f32x4 (&d)[2][4], f32x4 (&b)[4][NT], const uint32_t (&pix_off)[2][4],
    const uint32_t (&u_off)[4][NT], f32x16 (&acc)[4][NT], const __amdgpu_buffer_rsrc_t& srd_in, const __amdgpu_buffer_rsrc_t& srd_u,
    int next)
{
    // row XI of Bt over the patch rows, then Bt again over the columns
    f32x4 t[4], v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        t[j] = XI == 1 ? d[0][j] + d[1][j] : (XI == 2 ? d[1][j] - d[0][j] : d[0][j] - d[1][j]);
    v[0] = t[0] - t[2];
    v[1] = t[1] + t[2];
    v[2] = t[2] - t[1];
    v[3] = t[1] - t[3];
    __builtin_amdgcn_sched_barrier(0);
    if (AHEAD) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                d[r][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_in, (int)pix_off[r][j], next * 32, 0));
    }
#pragma unroll
    for (int nu = 0; nu < 4; ++nu) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                acc[nu][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(v[nu][e], b[nu][nt][e], acc[nu][nt], 0, 0, 0);
        if (AHEAD) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                b[nu][nt] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_u, (int)u_off[nu][nt], next * 16384, 0));
        }
        __builtin_amdgcn_sched_barrier(0); // (the scheduler would gather the loads at the end of the step, right before their use)
    }
}

// steps [step_begin, step_end) of a unit; the operands of step_begin have been requested (wino_load)
template <int NT, int XI>
__device__ __forceinline__ void wino_steps(f32x4 (&d)[2][4], f32x4 (&b)[4][NT], const uint32_t (&pix_off)[2][4],
    const uint32_t (&u_off)[4][NT], f32x16 (&acc)[4][NT], const __amdgpu_buffer_rsrc_t& srd_in, const __amdgpu_buffer_rsrc_t& srd_u,
    int step_begin, int step_end)
{
    for (int s = step_begin; s < step_end - 1; ++s)
        wino_step<NT, XI, true>(d, b, pix_off, u_off, acc, srd_in, srd_u, s + 1);
    wino_step<NT, XI, false>(d, b, pix_off, u_off, acc, srd_in, srd_u, 0);
}

// Persistent workgroups, balanced over the chip: the units of work (32 tiles x NT * 32 channels, cin / 8 steps each)
// form one line of steps, cut into as many equal stretches as there are workgroups.  A stretch that covers a unit
// from its first to its last step finishes it alone.  A unit that two or three stretches share is finished by the
// last of them to arrive: each leaves its share in the output domain (the transforms are linear, so shares add
// there) in the workspace with agent-scope stores, waits until they have left the CU, and takes the unit's ticket;
// the one that draws the last ticket adds all shares in stretch order (the result does not depend on who came last),
// then bias, residual and activation.  Nobody waits for anybody.  Without this a launch lasts a whole number of
// units per CU: 392 units on 256 CUs take the time of 512.
template <int NT>
__global__ __launch_bounds__(256, 2) void wino_kernel(WinoParams p)
{
    constexpr int NC = NT * 32, LS = NC + WINO_PAD;
    constexpr int LANES_PER_TILE = NC / 4, TILES_PER_PASS = 64 / LANES_PER_TILE, PASSES = WINO_TM / TILES_PER_PASS;
    constexpr int kAgentScope = 16; // cache-policy bit of a buffer access: written through to / fetched from memory
    extern __shared__ __attribute__((aligned(16))) float lds[]; // [4 rows][2][32 tiles][LS], then 32 tile descriptors
    __shared__ int last_flag;
    const int t = threadIdx.x, lane = t & 63, xi = t >> 6;
    const int fr = lane & 31, fh = lane >> 5;
    constexpr uint32_t OOB = 0x80000000u;
    const __amdgpu_buffer_rsrc_t srd_in = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.in), 0, (int)p.in_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_u = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.u), 0, (int)p.u_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_out = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, (int)p.out_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_res = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual ? p.residual : p.out), 0,
        (int)p.out_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t srd_ws = __builtin_amdgcn_make_buffer_rsrc(p.ws, 0, (int)p.ws_bytes, 0x00020000);
    int* tile_desc = reinterpret_cast<int*>(lds + 8 * WINO_TM * LS);
    const int oi = xi >> 1, oj = xi & 1; // the output pixel of every tile this wave finishes
    const int c4 = (lane % LANES_PER_TILE) * 4;
    constexpr uint32_t SHARE_BYTES = 4u * PASSES * 64u * 16u; // a unit's share in the workspace: [wave][pass][lane] 16-byte pieces

    // Workgroups are dealt to the eight XCDs in turn; stretch number g puts the workgroups of one XCD on neighbouring
    // stretches, and the units are ordered by column block first, so that an XCD's workgroups read the same slab of the
    // filter (which then stays in that XCD's L2) while each streams its own tiles.  With the tiles' order first, the
    // workgroups of an XCD were on all column blocks at once and the filter, 4-17 MB in the transform domain, was
    // fetched from memory once per unit.
    const int G = (int)gridDim.x;
    const int g = G % 8 == 0 ? ((int)blockIdx.x % 8) * (G / 8) + (int)blockIdx.x / 8 : (int)blockIdx.x;
    const int spu = p.cin / 8; // steps per unit
    // stretches: the first p.longer of them hold p.per_wg + 1 steps, the others p.per_wg (32-bit arithmetic throughout:
    // a 64-bit division costs more than a hundred instructions, and this runs once per unit)
    auto stretch_begin = [&](int gg) -> int { return gg * p.per_wg + (gg < p.longer ? gg : p.longer); };
    auto owner_of = [&](int step) -> int { // the stretch that holds `step`
        const int knee = p.longer * (p.per_wg + 1);
        return step < knee ? step / (p.per_wg + 1) : p.longer + (step - knee) / p.per_wg;
    };
    // a workgroup has two places in the workspace: one for the unit its stretch begins in, one for the unit it ends in
    auto share_off = [&](int gg, int unit) -> uint32_t {
        return (uint32_t)(2 * gg + (stretch_begin(gg) / spu == unit ? 0 : 1)) * SHARE_BYTES;
    };
    // What a lane needs to know of a unit: the offsets of its operands, and -- for the waves that finish the unit's
    // tiles -- where tile (lane % 32) goes: byte offset of its pixel (0, 0), channel 0, or an out-of-range offset; bit
    // 0 / 1 of the second word: the tile's second row / column exists.  A unit that is not live (there is none left
    // in the stretch) gives offsets that are out of range everywhere: loads from them return zeros and move nothing.
    struct UnitView {
        uint32_t pix_off[2][4], u_off[4][NT];
        int desc0, desc1;
    };
    const int end = stretch_begin(g + 1);
    auto view_of = [&](bool live, int unit, UnitView& v) {
        const int nb = (unit / (p.m_blocks * p.nb_group)) * p.nb_group + unit % p.nb_group;
        const int mb = (unit / p.nb_group) % p.m_blocks;
        // this lane's tile and the eight patch pixels row xi of Bt reads: rows (0, 2), (1, 2), (1, 2), (1, 3) of the patch
        const int tile = mb * WINO_TM + fr;
        const bool tile_ok = live && tile < p.tiles;
        const int rest = tile / p.tiles_x;
        const int tx = tile - rest * p.tiles_x;
        const int img = rest / p.tiles_y;
        const int ty = rest - img * p.tiles_y;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const int row = r == 0 ? (xi == 0 ? 0 : 1) : (xi == 0 ? 2 : (xi == 3 ? 3 : 2));
            const int y = 2 * ty - p.pad_top + row;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int x = 2 * tx - p.pad_left + j;
                const bool ok = tile_ok && y >= 0 && y < p.h && x >= 0 && x < p.w;
                v.pix_off[r][j] = ok ? (uint32_t)(((img * p.h + y) * p.w + x) * p.cin + fh * 4) * 4u : OOB;
            }
        }
#pragma unroll
        for (int nu = 0; nu < 4; ++nu)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
                v.u_off[nu][nt] = live ? (uint32_t)(((nb * NT + nt) * spu * 16 + xi * 4 + nu) * 64 + lane) * 16u : OOB;
        v.desc0 = tile_ok ? (int)((uint32_t)(((img * p.oh + 2 * ty) * p.ow + 2 * tx) * p.cout) * 4u) : (int)OOB;
        v.desc1 = (2 * ty + 1 < p.oh ? 1 : 0) | (2 * tx + 1 < p.ow ? 2 : 0);
    };
    f32x4 d[2][4], b[4][NT];
    UnitView cur;
    int pos = stretch_begin(g);
    int unit = pos / spu; // (the only division by the step count: from here on units are counted up)
    if (pos < end) {
        const int unit_begin = unit * spu;
        view_of(true, unit, cur);
        wino_load<NT>(d, b, cur.pix_off, cur.u_off, srd_in, srd_u, pos - unit_begin);
    }
    while (pos < end) {
        const int unit_begin = unit * spu;
        const int s0 = pos - unit_begin, s1 = end - unit_begin < spu ? end - unit_begin : spu;
        const int n0 = ((unit / (p.m_blocks * p.nb_group)) * p.nb_group + unit % p.nb_group) * NC;
        if (xi == 0 && fh == 0) {
            tile_desc[fr * 2] = cur.desc0;
            tile_desc[fr * 2 + 1] = cur.desc1;
        }

        f32x16 acc[4][NT];
#pragma unroll
        for (int nu = 0; nu < 4; ++nu)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[nu][nt][e] = 0.f;
        switch (xi) { // the row of Bt is a compile-time choice inside the loop
        case 0: wino_steps<NT, 0>(d, b, cur.pix_off, cur.u_off, acc, srd_in, srd_u, s0, s1); break;
        case 1: wino_steps<NT, 1>(d, b, cur.pix_off, cur.u_off, acc, srd_in, srd_u, s0, s1); break;
        case 2: wino_steps<NT, 2>(d, b, cur.pix_off, cur.u_off, acc, srd_in, srd_u, s0, s1); break;
        default: wino_steps<NT, 3>(d, b, cur.pix_off, cur.u_off, acc, srd_in, srd_u, s0, s1); break;
        }
        // the next unit's first operands set out now and travel while this unit's results are exchanged and stored
        const int next_pos = unit_begin + s1; // the next unit begins at its first step
        {
            const bool live = next_pos < end;
            view_of(live, unit + 1, cur);
            wino_load<NT>(d, b, cur.pix_off, cur.u_off, srd_in, srd_u, 0);
        }

        // At along the row: z0 = m0 + m1 + m2, z1 = m1 - m2 - m3.  Element e of a lane is tile 8 * (e / 4) + 4 * fh +
        // e % 4, channel nt * 32 + fr.
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = 8 * (e / 4) + 4 * fh + (e % 4);
                const float m1 = acc[1][nt][e], m2 = acc[2][nt][e];
                lds[((xi * 2 + 0) * WINO_TM + row) * LS + nt * 32 + fr] = acc[0][nt][e] + m1 + m2;
                lds[((xi * 2 + 1) * WINO_TM + row) * LS + nt * 32 + fr] = m1 - m2 - acc[3][nt][e];
            }
        __syncthreads();

        // At along the column: wave (oi, oj) combines the rows into its pixel of every tile
        auto combine = [&](int pass) -> f32x4 {
            const int tl = pass * TILES_PER_PASS + lane / LANES_PER_TILE;
            const float* z = lds + (oj * WINO_TM + tl) * LS + c4; // row 0 of the domain, column value oj
            const f32x4 za = *reinterpret_cast<const f32x4*>(z + (oi == 0 ? 0 : 1) * 2 * WINO_TM * LS);
            const f32x4 zb = *reinterpret_cast<const f32x4*>(z + (oi == 0 ? 1 : 2) * 2 * WINO_TM * LS);
            const f32x4 zc = *reinterpret_cast<const f32x4*>(z + (oi == 0 ? 2 : 3) * 2 * WINO_TM * LS);
            return oi == 0 ? za + zb + zc : za - zb - zc;
        };
        f32x4 bias4 = { 0.f, 0.f, 0.f, 0.f };
        if (p.bias)
            bias4 = *reinterpret_cast<const f32x4*>(p.bias + n0 + c4);
        auto finish = [&](int pass, f32x4 y) {
            const int tl = pass * TILES_PER_PASS + lane / LANES_PER_TILE;
            const int base = tile_desc[tl * 2], flags = tile_desc[tl * 2 + 1];
            const bool ok = (oi == 0 || (flags & 1)) && (oj == 0 || (flags & 2));
            const uint32_t off = ok ? (uint32_t)base + (uint32_t)((oi * p.ow + oj) * p.cout + n0 + c4) * 4u : OOB;
            y += bias4;
            if (p.residual)
                y += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_res, (int)off, 0, 0));
            float v[4] = { y[0], y[1], y[2], y[3] };
            apply_act_block(v, p.act);
            const f32x4 r = { v[0], v[1], v[2], v[3] };
            // (agent scope: written through to memory instead of left dirty in this XCD's L2 until the kernel ends)
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, r), srd_out, (int)off, 0, kAgentScope);
        };
        if (s0 == 0 && s1 == spu) {
#pragma unroll 4
            for (int pass = 0; pass < PASSES; ++pass)
                finish(pass, combine(pass));
        } else {
            const uint32_t lane_off = (uint32_t)((xi * PASSES) * 64 + lane) * 16u;
            const uint32_t mine = share_off(g, unit) + lane_off;
            const int g_a = owner_of(unit_begin), parts = owner_of(unit_begin + spu - 1) - g_a + 1;
            // A stretch that ends inside this unit comes to it at the very end of its life; the stretches that hold the
            // unit's later steps began with them and handed their shares in long ago.  One look at the ticket then shows
            // everybody else in -- each took its ticket after its share had left its CU -- and this workgroup, certainly
            // the last, neither stores a share of its own nor draws a ticket: two trips to memory fewer at the one place
            // where nothing else is left to run beside them.
            bool finish_here = false;
            if (s1 < spu) {
                if (t == 0)
                    last_flag = __hip_atomic_load(p.tickets + unit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == parts - 1;
                __syncthreads();
                finish_here = last_flag != 0;
                __syncthreads(); // last_flag is written again below
            }
            if (finish_here) {
                if (t == 0)
                    __hip_atomic_store(p.tickets + unit, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // for the next launch
            } else {
#pragma unroll 4
                for (int pass = 0; pass < PASSES; ++pass)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, combine(pass)), srd_ws, (int)(mine + (uint32_t)pass * 1024u),
                        0, kAgentScope);
                // every lane's share has left the CU before the ticket is taken
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (t == 0) {
                    const int ticket = __hip_atomic_fetch_add(p.tickets + unit, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const int last = ticket == parts - 1;
                    if (last)
                        __hip_atomic_store(p.tickets + unit, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // for the next launch
                    last_flag = last;
                }
                __syncthreads();
                finish_here = last_flag != 0;
            }
            if (finish_here) {
                // shares are added in stretch order whoever came last; this workgroup's own one is formed again from the
                // exchange area (the same operations on the same values, so the same bits) instead of read back
                const int my_part = g - g_a;
                for (int pass = 0; pass < PASSES; ++pass) {
                    f32x4 y = { 0.f, 0.f, 0.f, 0.f };
                    for (int sp = 0; sp < parts; ++sp) {
                        if (sp == my_part)
                            y += combine(pass);
                        else
                            y += __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_ws,
                                (int)(share_off(g_a + sp, unit) + lane_off + (uint32_t)pass * 1024u), 0, kAgentScope));
                    }
                    finish(pass, y);
                }
            }
        }
        __syncthreads(); // the next unit overwrites the exchange area, the tile descriptors and last_flag
        pos = next_pos;
        ++unit;
    }
}

static size_t wino_lds_bytes(int nt) { return sizeof(float) * (size_t)8 * WINO_TM * (nt * 32 + WINO_PAD) + sizeof(int) * 2 * WINO_TM; }

// library-owned scratch: two shares of 32 KB per workgroup of the persistent grid, one ticket per unit (zero
// between launches: the workgroup that finishes a unit resets its ticket)
constexpr int kWinoTickets = 1 << 16;
constexpr size_t kWinoShareBytes = 32 * 1024;
static float* g_wino_ws = nullptr;
static int* g_wino_tickets = nullptr;
static int g_wino_grid = 0;

static bool wino_prepare()
{
    static std::mutex mu;
    std::lock_guard<std::mutex> lock(mu);
    if (g_wino_ws && g_wino_tickets)
        return true;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess || prop.multiProcessorCount < 1)
        return false;
    g_wino_grid = 2 * prop.multiProcessorCount; // at most two workgroups per CU
    if (!g_wino_ws && hipMalloc(&g_wino_ws, 2 * kWinoShareBytes * (size_t)g_wino_grid) != hipSuccess)
        return false;
    if (!g_wino_tickets
        && (hipMalloc(&g_wino_tickets, sizeof(int) * kWinoTickets) != hipSuccess
            || zero_device(g_wino_tickets, sizeof(int) * kWinoTickets) != hipSuccess))
        return false;
    return true;
}

static bool al16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15) == 0; }

} // namespace fdx

using namespace fdx;

extern "C" int fdx_conv2d_winograd_supported(int cin, int cout)
{
    return cin > 0 && cin % 8 == 0 && cout > 0 && cout % 64 == 0;
}

extern "C" size_t fdx_conv2d_winograd_weight_floats(int cout, int cin) { return (size_t)16 * (size_t)cout * (size_t)cin; }

// (G g Gt)[a][b] for the 3x3 filter g of every (cout, cin), in the order the kernel's lanes take it:
// u[cout / 32][cin / 8][p = 4 a + b][32 * (cin % 8 / 4) + cout % 32][cin % 4]; host memory on both sides
extern "C" fdx_status fdx_conv2d_winograd_prepare(const float* weights_nkkc, int cout, int cin, float* u_out)
{
    FDX_REQUIRE(weights_nkkc && u_out && fdx_conv2d_winograd_supported(cin, cout), "winograd_prepare: bad arguments");
    static const double G[4][3] = { { 1.0, 0.0, 0.0 }, { 0.5, 0.5, 0.5 }, { 0.5, -0.5, 0.5 }, { 0.0, 0.0, 1.0 } };
    const size_t steps = (size_t)cin / 8;
    for (int n = 0; n < cout; ++n)
        for (int c = 0; c < cin; ++c) {
            double g[3][3], gg[4][3];
            for (int y = 0; y < 3; ++y)
                for (int x = 0; x < 3; ++x)
                    g[y][x] = weights_nkkc[(((size_t)n * 3 + y) * 3 + x) * cin + c];
            for (int a = 0; a < 4; ++a)
                for (int x = 0; x < 3; ++x)
                    gg[a][x] = G[a][0] * g[0][x] + G[a][1] * g[1][x] + G[a][2] * g[2][x];
            const size_t lane = (size_t)32 * ((c % 8) / 4) + n % 32;
            for (int a = 0; a < 4; ++a)
                for (int b = 0; b < 4; ++b)
                    u_out[(((((size_t)n / 32) * steps + c / 8) * 16 + (a * 4 + b)) * 64 + lane) * 4 + c % 4]
                        = (float)(gg[a][0] * G[b][0] + gg[a][1] * G[b][1] + gg[a][2] * G[b][2]);
        }
    return FDX_OK;
}

// a size the kernel's 32-bit offsets and tickets do not cover: not an error of the caller, who has the direct kernel
#define FDX_WINO_LIMIT(cond, ...)                                                                         \
    do {                                                                                                  \
        if (!(cond)) {                                                                                    \
            fdx::set_error(__VA_ARGS__);                                                                  \
            return FDX_ERR_UNSUPPORTED;                                                                   \
        }                                                                                                 \
    } while (0)

extern "C" fdx_status fdx_conv2d_winograd_nhwc_f32(const float* in, int n, int h, int w, int cin, const float* u_weights, const float* bias,
    int cout, int pad_top, int pad_left, int out_h, int out_w, const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && u_weights && out, "conv2d_winograd: null pointer");
    FDX_REQUIRE(n > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0, "conv2d_winograd: bad shape");
    if (!fdx_conv2d_winograd_supported(cin, cout)) {
        set_error("conv2d_winograd: needs input channels %% 8 == 0 and output channels %% 64 == 0");
        return FDX_ERR_UNSUPPORTED;
    }
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(al16(in) && al16(u_weights) && al16(out) && (!bias || al16(bias)) && (!residual || al16(residual)),
        "conv2d_winograd: operands must be 16-byte aligned");
    FDX_REQUIRE(pad_top >= 0 && pad_left >= 0 && out_h - 1 - pad_top < h && out_w - 1 - pad_left < w,
        "conv2d_winograd: output size does not fit the input");
    WinoParams p;
    std::memset(&p, 0, sizeof p);
    p.in = in; p.u = u_weights; p.bias = bias; p.residual = residual; p.out = out;
    p.n = n; p.h = h; p.w = w; p.cin = cin; p.cout = cout; p.pad_top = pad_top; p.pad_left = pad_left; p.oh = out_h; p.ow = out_w;
    p.tiles_x = (out_w + 1) / 2;
    p.tiles_y = (out_h + 1) / 2;
    FDX_WINO_LIMIT((int64_t)n * p.tiles_x * p.tiles_y < (1LL << 30), "conv2d_winograd: too many output pixels for one launch");
    p.tiles = n * p.tiles_x * p.tiles_y;
    FDX_WINO_LIMIT((int64_t)n * h * w * cin * 4 < (1LL << 31), "conv2d_winograd: input tensor beyond 2 GiB");
    p.in_bytes = (uint32_t)((int64_t)n * h * w * cin * 4);
    FDX_WINO_LIMIT((int64_t)n * out_h * out_w * cout * 4 < (1LL << 31), "conv2d_winograd: output tensor beyond 2 GiB");
    p.out_bytes = (uint32_t)((int64_t)n * out_h * out_w * cout * 4);
    FDX_WINO_LIMIT((int64_t)16 * cout * cin * 4 < (1LL << 31), "conv2d_winograd: filter beyond 2 GiB");
    p.u_bytes = (uint32_t)((int64_t)16 * cout * cin * 4);
    p.act = make_act(act);
    FDX_REQUIRE(wino_prepare(), "conv2d_winograd: no device memory for the workspace");
    const int m_blocks = (p.tiles + WINO_TM - 1) / WINO_TM;
    // (128-channel units -- NT = 4, 256 accumulators, one workgroup per CU -- were measured: half the patch loads per
    // MFMA, but 14x14 256 -> 256 takes 110 us instead of 87: half as many units, so every one is cut by a stretch
    // boundary, and the exchange at a unit's end is twice as long with nothing beside it on the SIMD)
    constexpr int nt = 2;
    p.m_blocks = m_blocks;
    p.n_blocks = cout / (nt * 32);
    if ((int64_t)m_blocks * p.n_blocks > kWinoTickets) {
        set_error("conv2d_winograd: more than %d units of work in one launch", kWinoTickets);
        return FDX_ERR_UNSUPPORTED;
    }
    p.units = m_blocks * p.n_blocks;
    // Column block first keeps one slab of the filter in an XCD's L2, at the price of the input crossing the fabric once
    // per column block.  Column blocks whose slabs together stay within 2 MB (half an L2) form a group that shares the
    // walk over the tile blocks: inside a group a tile block's column blocks follow each other, and the input is
    // fetched once per group (128 -> 128 channels: one group, the tiles' order first; 256 -> 256: two groups of two;
    // 512 -> 512: every column block on its own).
    static const bool lean = [] { const char* e = std::getenv("FDX_WINO_ORDER"); return !(e && e[0] == '0'); }();
    const size_t slab_bytes = fdx_conv2d_winograd_weight_floats(cin, cout) * sizeof(float) / (size_t)p.n_blocks;
    p.nb_group = 1;
    if (lean)
        for (int gsz = 2; gsz <= p.n_blocks; ++gsz)
            if (p.n_blocks % gsz == 0 && (size_t)gsz * slab_bytes <= ((size_t)2 << 20))
                p.nb_group = gsz;
    p.ws = g_wino_ws;
    p.ws_bytes = (uint32_t)(2 * kWinoShareBytes * (size_t)g_wino_grid);
    p.tickets = g_wino_tickets;
    // every workgroup gets at least four steps; none gets an empty stretch
    const int64_t total_steps = (int64_t)p.units * (cin / 8);
    FDX_WINO_LIMIT(total_steps < (1LL << 30), "conv2d_winograd: too many steps for one launch");
    const int64_t by_steps = total_steps / 4 > 0 ? total_steps / 4 : 1;
    // Two workgroups fit on a CU.  The second one pays where units are short (64 input channels: 8 steps per unit, -9 %;
    // 128: -3 %): the end of one's unit runs under the other's steps.  Units of 32 and 64 steps gain nothing there and
    // lose 2-8 % to the shares of the units that twice as many stretches cut: one workgroup per CU for them.  (The
    // steps themselves do not get faster with a second wave on the SIMD: their loads -- 16 per 32 MFMAs, the patch
    // pieces 32 lines per instruction -- keep the CU's vector memory path as busy as the MFMAs keep the matrix pipe.)
    const int resident = cin <= 128 ? g_wino_grid : g_wino_grid / 2;
    const dim3 grid((unsigned)(by_steps < resident ? by_steps : resident));
    p.per_wg = (int)(total_steps / grid.x);
    p.longer = (int)(total_steps % grid.x);
    const size_t lds = wino_lds_bytes(nt);
    profile_begin();
    static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(wino_kernel<2>),
        hipFuncAttributeMaxDynamicSharedMemorySize, (int)wino_lds_bytes(2));
    FDX_WINO_LIMIT(attr == hipSuccess, "conv2d_winograd: the kernel's LDS request was refused");
    hipLaunchKernelGGL(wino_kernel<2>, grid, dim3(256), lds, stream(), p);
    const double pix = (double)n * out_h * out_w;
    const double tiles = (double)n * ((out_h + 1) / 2) * ((out_w + 1) / 2);
    profile_end("conv2d_winograd_f32", 2.0 * pix * 9.0 * cin * cout, 4.0 * ((double)n * h * w * cin + pix * cout * (residual ? 2.0 : 1.0) + 9.0 * cin * cout),
        2.0 * 16.0 * tiles * cin * cout);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

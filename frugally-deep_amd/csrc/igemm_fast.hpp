// Fast path of the implicit-GEMM Conv2D / GEMM (included inside namespace fdx by igemm.hip).
//
// Same tiling and MFMA schedule as igemm_kernel, with the per-slab overhead stripped for the
// shapes that dominate real networks (Cin, or K for a plain GEMM, a multiple of the slab; N a
// multiple of 4), and the workgroups made persistent:
//
//  * Operands are fetched with raw buffer loads: each lane keeps ONE 32-bit byte offset per
//    tile row for the whole K loop, the walk along K is a scalar offset shared by the
//    workgroup (filter tap and channel are uniform within a slab), and a padded or
//    out-of-range tap is an offset beyond the buffer's extent, which the hardware answers
//    with zeros -- no branches, no per-slab address arithmetic.  A's base is shifted down by
//    the top-left padding so offsets stay non-negative.
//  * A workgroup walks a strided list of output tiles.  Before it writes a finished tile it
//    already has the first slab of its next tile in flight, and the tile's stores drain while
//    the next tile computes: output traffic and first-load latency overlap with MFMA work
//    instead of adding to it (with one tile per workgroup all workgroups of a round reach
//    their epilogue together and the matrix cores idle while HBM drains).
//  * The epilogue goes through LDS so that bias, residual and output move as 16-byte
//    accesses along the channel axis.
//  * SPLIT: a layer with too few output tiles for the chip (late stages of a CNN at small
//    batch) cuts every tile's K range into `splits` units.  A unit leaves its accumulators in a
//    workspace and takes a ticket on the tile; the last unit to arrive adds all partial tiles
//    in split order (so the sum does not depend on arrival order) and runs the epilogue.
//    Nothing waits on another workgroup.  Partials are written and read with agent-scope
//    accesses, which pass the per-XCD L2s, instead of a fence that writes a whole L2 back.
//  * SPLIT with splits == 0 ("stream-K"): the slabs of all tiles form one line that is cut into
//    as many equal pieces as there are workgroups, so every workgroup does the same amount of
//    MFMA work whatever the tile count.  A workgroup's piece covers the end of one tile, some
//    whole tiles and the beginning of another; the (at most two) partial tiles go through the
//    same workspace / ticket / ordered-sum path, with the number of contributors of a tile
//    and their workspace slots computed from the cut points.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

//  * DUAL (GEMM form, whole tiles only): the rows of A come from two tensors -- the first K1 columns from A with row
//    stride lda, the other K - K1 from A2, whose row for output pixel (image, y, x) is pixel (y * s2y, x * s2x) of an
//    [H2][W2][C2] map.  That is the sum of two pointwise convolutions as one GEMM over the concatenated channels
//    (a residual block whose shortcut is a 1x1 convolution: the shortcut's output is never written or read back).
//  * LNF (GEMM form, whole tiles only, K = the whole row): the rows of A are layer-normalised over K on the way,
//        C = act(LN(A) . B^T + bias)  with  LN(a) = (a - mean) / sqrt(var + eps)   (gamma folded into B, beta into bias
//    by the caller; include/fdeep/layers/layer_normalization_layer.hpp:37-63).  A tile's K loop reads its rows from end
//    to end anyway, so the row statistics are gathered from the operand registers on their way to LDS (sums of the
//    differences to the row's first value a thread sees, which keeps them small whatever the row's mean), merged over
//    the lanes that share a row after the loop, and applied in the epilogue as
//        rstd * (acc - mean * rowsum(B)) + bias:
//    no pass over A of its own, and the normalised tensor never exists.
template <int BM, int BN, int WAVES_M, int WAVES_N, int BKT, bool CONV, bool SPLIT = false, bool STREAMK = false, bool DUAL = false,
    bool LNF = false>
// (the second bound asks for two waves per SIMD where the split variant of the largest four-wave tile would otherwise
// settle for one: its reduction holds the accumulators in ordinary registers next to the prefetched operands)
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, (SPLIT && WAVES_M * WAVES_N == 4 && BM * BN >= 128 * 128) ? 2 : 1)
void igemm_fast_kernel(GemmParams p)
{
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    static_assert(NT == 256 || NT == 512, "four or eight waves");
    static_assert(!DUAL || (!CONV && !SPLIT), "the two-source form is a whole-tile GEMM");
    static_assert(!LNF || (!CONV && !SPLIT && !DUAL), "the normalising form is a whole-tile GEMM");
    constexpr int STRIDE = BKT + 4;
    constexpr int CPR = BKT / 4;  // 16-byte chunks per tile row
    constexpr int RPP = NT / CPR; // tile rows filled per loader pass
    constexpr int A_LOADS = BM / RPP, B_LOADS = BN / RPP;
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows must be a multiple of the loader pass");
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int OSTRIDE = WTN + 4; // epilogue scratch row
    static_assert(2 * (BM + BN) * STRIDE >= WAVES_M * WAVES_N * 32 * OSTRIDE, "epilogue scratch must fit in the operand buffers");
    constexpr uint32_t OOB = 0x80000000u; // beyond any extent this path accepts: the load returns zeros

    __shared__ __attribute__((aligned(16))) float smem[2 * (BM + BN) * STRIDE];
    __shared__ int last_flag;
    __shared__ float ln_stats[LNF ? 2 * BM : 2]; // (mean, 1 / sqrt(var + eps)) per tile row

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int kq = t % CPR, r0 = t / CPR;
    const int fr = lane & 31, fh = lane >> 5;

    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    const int per_problem = tiles_m * tiles_n;
    const int S = SPLIT ? p.splits : 1;
    const int all_tiles = per_problem * p.batch;
    // Units of work: the first n_dp tiles are computed whole; every later tile is cut into S K ranges ("split
    // units").  XCD x (workgroups with blockIdx % 8 == x) owns a contiguous range of the whole tiles and one of the
    // split units, so tiles that share an A row block also share that XCD's L2 and both kinds of work are spread
    // evenly; its workgroups stride through the two ranges one after the other.
    const int n_dp = SPLIT ? p.split_dp_tiles : all_tiles, n_su = SPLIT ? (all_tiles - n_dp) * S : 0;
    const int xcd = blockIdx.x & 7, wg_in_xcd = blockIdx.x >> 3;
    const int wgs_in_xcd = ((int)gridDim.x - xcd + 7) >> 3;
    const int alo = xcd * (n_dp >> 3) + (xcd < (n_dp & 7) ? xcd : (n_dp & 7)), na = (n_dp >> 3) + (xcd < (n_dp & 7) ? 1 : 0);
    const int blo = xcd * (n_su >> 3) + (xcd < (n_su & 7) ? xcd : (n_su & 7)), nb = (n_su >> 3) + (xcd < (n_su & 7) ? 1 : 0);
    const int hi = na + nb; // local unit indices [0, hi)
    const int KT = p.K / BKT;

    // stream-K: workgroup g (numbered XCD by XCD, so an XCD owns a contiguous stretch of tiles) takes the slabs
    // [g * W / G, (g + 1) * W / G) of the W = tiles * KT slabs; its units are the tiles that stretch touches
    // (a template argument: carried as a run-time flag, the extra index arithmetic cost the plain split variant a
    // tenth of its speed)
    static_assert(!STREAMK || SPLIT, "stream-K is a form of the split variant");
    constexpr bool sk = STREAMK;
    const int G = (int)gridDim.x;
    const int g_lin = xcd * (G >> 3) + (xcd < (G & 7) ? xcd : (G & 7)) + wg_in_xcd;
    const int64_t W = (int64_t)all_tiles * KT;
    const int64_t sk_lo = sk ? g_lin * W / G : 0, sk_hi = sk ? (g_lin + 1) * W / G : 0;
    const int sk_first = sk ? (int)(sk_lo / KT) : 0;
    const int sk_units = (sk && sk_hi > sk_lo) ? (int)((sk_hi - 1) / KT) - sk_first + 1 : 0;

    // ---- per-tile loader state
    uint32_t a_voff[A_LOADS], b_voff[B_LOADS];
    uint32_t a2_voff[DUAL ? A_LOADS : 1];
    uint64_t a_mask[A_LOADS];
    __amdgpu_buffer_rsrc_t srd_a, srd_b;
    const __amdgpu_buffer_rsrc_t srd_a2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(DUAL ? p.A2 : p.A), 0,
        DUAL ? (int)p.a2_records : 0, 0x00020000);
    int tap, fx, fy, c0, soff_a, soff_b;
    f32x4 ra[A_LOADS], rb[B_LOADS];
    int kt_n = KT; // slabs of the current unit

    int cur_su = -1;  // workspace slot of the current work item's partial tile, -1 for a whole tile
    int cur_tile = 0; // its output tile
    auto setup = [&](int local, int& m0, int& n0, int64_t& c_off) {
        int tile = alo + local, kt_lo = 0;
        cur_su = -1;
        kt_n = KT;
        if (sk) {
            tile = sk_first + local;
            const int64_t t0 = (int64_t)tile * KT;
            kt_lo = sk_lo > t0 ? (int)(sk_lo - t0) : 0;
            const int kt_hi = sk_hi - t0 < KT ? (int)(sk_hi - t0) : KT;
            kt_n = kt_hi - kt_lo;
            // a workgroup leaves at most two partial tiles: one that began before its stretch (slot 2g) and one that
            // ends after it (slot 2g + 1)
            if (kt_n < KT)
                cur_su = 2 * g_lin + (sk_lo > t0 ? 0 : 1);
        } else if (SPLIT && local >= na) {
            cur_su = blo + (local - na);
            tile = n_dp + cur_su / S;
            const int split = cur_su - (cur_su / S) * S;
            kt_lo = (int)((int64_t)split * KT / S);
            kt_n = (int)((int64_t)(split + 1) * KT / S) - kt_lo;
        }
        cur_tile = tile;
        const int z = tile / per_problem, id = tile - z * per_problem;
        if (p.strip_w > 0) {
            const int per_strip = tiles_m * p.strip_w, last = (tiles_n - 1) / p.strip_w;
            int strip = id / per_strip;
            strip = strip < last ? strip : last; // the last strip may be narrower
            const int rem = id - strip * per_strip, left = tiles_n - strip * p.strip_w;
            const int w_eff = p.strip_w < left ? p.strip_w : left;
            const int mt = rem / w_eff;
            m0 = mt * BM;
            n0 = (strip * p.strip_w + (rem - mt * w_eff)) * BN;
        } else {
            m0 = (id / tiles_n) * BM;
            n0 = (id % tiles_n) * BN;
        }
        const float* A = p.A + (z / p.inner) * p.a_outer + (z % p.inner) * p.a_inner;
        const float* B = p.B + (z / p.inner) * p.b_outer + (z % p.inner) * p.b_inner;
        c_off = (z / p.inner) * p.c_outer + (z % p.inner) * p.c_inner;
        srd_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(A), 0, (int)p.a_records, 0x00020000);
        srd_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(B), 0, (int)p.b_records, 0x00020000);
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int m = m0 + r0 + i * RPP;
            a_voff[i] = OOB;
            a_mask[i] = 0;
            if (m < p.M) {
                if (CONV) {
                    const int img = m / (p.OH * p.OW), rm = m - img * (p.OH * p.OW);
                    const int oy = rm / p.OW, ox = rm - oy * p.OW;
                    const int iy0 = oy * p.sy - p.pad_top, ix0 = ox * p.sx - p.pad_left;
                    // byte offset from the shifted base (shift = (pad_top*W + pad_left)*Cin elements)
                    a_voff[i] = (uint32_t)(((img * p.H + oy * p.sy) * p.W + ox * p.sx) * p.pix_stride) * 4u + kq * 16;
                    uint64_t mk = 0;
                    for (int y = 0; y < p.kh; ++y) {
                        const int iy = iy0 + y * p.dy;
                        for (int x = 0; x < p.kw; ++x) {
                            const int ix = ix0 + x * p.dx;
                            if (iy >= 0 && iy < p.H && ix >= 0 && ix < p.W)
                                mk |= 1ull << (y * p.kw + x);
                        }
                    }
                    a_mask[i] = mk;
                } else {
                    a_voff[i] = (uint32_t)((int64_t)m * p.lda) * 4u + kq * 16;
                    a_mask[i] = ~0ull;
                }
            }
            if (DUAL) {
                a2_voff[i] = OOB;
                if (m < p.M) {
                    const int img = m / (p.OH * p.OW), rm = m - img * (p.OH * p.OW);
                    const int oy = rm / p.OW, ox = rm - oy * p.OW;
                    a2_voff[i] = (uint32_t)(((img * p.H2 + oy * p.s2y) * p.W2 + ox * p.s2x) * p.C2) * 4u + kq * 16;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const int n = n0 + r0 + i * RPP;
            b_voff[i] = n < p.N ? (uint32_t)((int64_t)n * p.ldb) * 4u + kq * 16 : OOB;
        }
        tap = fx = fy = c0 = 0;
        soff_a = soff_b = 0;
        if (SPLIT && kt_lo > 0) {
            const int k_start = kt_lo * BKT;
            soff_b = k_start * 4;
            if (CONV) {
                tap = k_start / p.Cin;
                c0 = k_start - tap * p.Cin;
                fy = tap / p.kw;
                fx = tap - fy * p.kw;
                soff_a = ((fy * p.dy * p.W + fx * p.dx) * p.pix_stride + c0) * 4;
            } else {
                soff_a = k_start * 4;
            }
        }
    };
    auto load_tiles = [&]() {
        if (DUAL && soff_b >= p.K1 * 4) { // the slab lies in the second tensor's columns (uniform over the workgroup)
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i)
                ra[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_a2, (int)a2_voff[DUAL ? i : 0], soff_b - p.K1 * 4, 0));
        } else {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const uint32_t vo = CONV ? (((a_mask[i] >> tap) & 1) ? a_voff[i] : OOB) : a_voff[i];
                ra[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_a, (int)vo, soff_a, 0));
            }
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i)
            rb[i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(srd_b, (int)b_voff[i], soff_b, 0));
        soff_b += BKT * 4;
        if (CONV) {
            c0 += BKT;
            if (c0 == p.Cin) {
                c0 = 0;
                ++tap;
                if (++fx == p.kw) {
                    fx = 0;
                    ++fy;
                }
            }
            soff_a = ((fy * p.dy * p.W + fx * p.dx) * p.pix_stride + c0) * 4;
        } else {
            soff_a += BKT * 4;
        }
    };
    float ln_shift[LNF ? A_LOADS : 1], ln_s[LNF ? A_LOADS : 1], ln_q[LNF ? A_LOADS : 1];
    auto store_tiles = [&](int buf, bool first = false) {
        float* as = smem + buf * (BM + BN) * STRIDE;
        float* bs = as + BM * STRIDE;
        if (LNF) {
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                if (first) {
                    ln_shift[LNF ? i : 0] = ra[i][0];
                    ln_s[LNF ? i : 0] = 0.f;
                    ln_q[LNF ? i : 0] = 0.f;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float dlt = ra[i][e] - ln_shift[LNF ? i : 0];
                    ln_s[LNF ? i : 0] += dlt;
                    ln_q[LNF ? i : 0] += dlt * dlt;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            *reinterpret_cast<f32x4*>(&as[(r0 + i * RPP) * STRIDE + kq * 4]) = ra[i];
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i)
            *reinterpret_cast<f32x4*>(&bs[(r0 + i * RPP) * STRIDE + kq * 4]) = rb[i];
    };

    int tile = sk ? 0 : wg_in_xcd; // local unit index
    const int unit_step = sk ? 1 : wgs_in_xcd, unit_end = sk ? sk_units : hi;
    if (tile >= unit_end)
        return; // uniform per workgroup
    int m0, n0;
    int64_t c_off;
    setup(tile, m0, n0, c_off);
    load_tiles();

    for (;;) {
        f32x16 acc[TM][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    acc[i][j][e] = 0.f;

        store_tiles(0, true);
        __syncthreads();
        const int kt_end = kt_n;
        for (int kt = 0; kt < kt_end; ++kt) {
            const int buf = kt & 1;
            if (kt + 1 < kt_end)
                load_tiles();
            const float* as = smem + buf * (BM + BN) * STRIDE;
            const float* bs = as + BM * STRIDE;
            if (TM == 1 && TN == 1) {
                // one 32 x 32 piece per wave: the fragments of the whole slab are requested from LDS before the first MFMA
                // (read two groups at a time, the second pair of groups waited out its LDS latency with the pipe drained: the
                // encoder's GEMMs 1 % faster this way)
                f32x4 af[BKT / 8], bf[BKT / 8];
#pragma unroll
                for (int k8 = 0; k8 < BKT / 8; ++k8) {
                    af[k8] = *reinterpret_cast<const f32x4*>(&as[(wm * WTM + fr) * STRIDE + k8 * 8 + fh * 4]);
                    bf[k8] = *reinterpret_cast<const f32x4*>(&bs[(wn * WTN + fr) * STRIDE + k8 * 8 + fh * 4]);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int k8 = 0; k8 < BKT / 8; ++k8)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[k8][e], bf[k8][e], acc[0][0], 0, 0, 0);
            } else {
#pragma unroll
            for (int k8 = 0; k8 < BKT / 8; ++k8) {
                f32x4 af[TM], bf[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    af[i] = *reinterpret_cast<const f32x4*>(&as[(wm * WTM + i * 32 + fr) * STRIDE + k8 * 8 + fh * 4]);
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    bf[j] = *reinterpret_cast<const f32x4*>(&bs[(wn * WTN + j * 32 + fr) * STRIDE + k8 * 8 + fh * 4]);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][e], bf[j][e], acc[i][j], 0, 0, 0);
            }
            }
            if (kt + 1 < kt_end)
                store_tiles(buf ^ 1);
            if (LNF && kt + 1 == kt_end) {
                // Every slab has passed through store_tiles by now, so every thread has seen 4 * KT values of each of its
                // rows.  The eight lanes that share a row (consecutive lanes, CPR = 8) merge their means and sums of
                // squared deviations pairwise, equal counts on both sides at every step, on the VALU's lane swaps: inside
                // quads twice, then with the mirrored lane of the row's eight, whose quad holds the other half's result.
                // Done here, behind the last slab's MFMAs and in front of the loop's last barrier, it costs no barrier of
                // its own.
                static_assert(!LNF || CPR == 8, "the merge below is written for eight lanes per row");
#pragma unroll
                for (int i = 0; i < A_LOADS; ++i) {
                    float cnt = 4.0f * (float)KT;
                    float mean = ln_shift[LNF ? i : 0] + ln_s[LNF ? i : 0] / cnt;
                    float m2 = ln_q[LNF ? i : 0] - ln_s[LNF ? i : 0] * ln_s[LNF ? i : 0] / cnt;
                    auto merge = [&](float om, float o2) {
                        const float dlt = om - mean;
                        mean = 0.5f * (mean + om);
                        m2 = m2 + o2 + dlt * dlt * (0.5f * cnt);
                        cnt *= 2.0f;
                    };
                    merge(dpp_move<0xB1>(mean), dpp_move<0xB1>(m2));   // quad_perm [1, 0, 3, 2]
                    merge(dpp_move<0x4E>(mean), dpp_move<0x4E>(m2));   // quad_perm [2, 3, 0, 1]
                    merge(dpp_move<0x141>(mean), dpp_move<0x141>(m2)); // row_half_mirror
                    if (kq == 0) {
                        ln_stats[2 * (r0 + i * RPP)] = mean;
                        ln_stats[2 * (r0 + i * RPP) + 1] = 1.0f / sqrtf(fmaxf(m2, 0.f) / cnt + p.ln_eps);
                    }
                }
            }
            __syncthreads();
        }


        // this tile's coordinates for the epilogue; the loader state moves on to the next tile
        const int em0 = m0, en0 = n0;
        float* __restrict__ C = p.C + c_off;
        const float* __restrict__ R = p.residual ? p.residual + c_off : nullptr;
        const int su_done = cur_su, tile_done = cur_tile;
        // What the epilogue reads from memory -- the bias and the residual rows of the first 32-row band -- is requested
        // before the next tile's operands: loads complete in the order of their issue, so behind those operands their
        // first use would wait for the whole prefetch.
        constexpr int LPR = WTN / 4;  // lanes per scratch row
        constexpr int RPS = 64 / LPR; // rows per store pass
        const int srow = lane / LPR, scol = (lane % LPR) * 4;
        const int n = en0 + wn * WTN + scol;
        const bool n_ok = n < p.N; // N is a multiple of 4 on this path
        f32x4 bias4 = { 0.f, 0.f, 0.f, 0.f };
        f32x4 rr[32 / RPS];
        auto request_residual = [&](int i) {
#pragma unroll
            for (int ps = 0; ps < 32 / RPS; ++ps) {
                const int m = em0 + wm * WTM + i * 32 + ps * RPS + srow;
                rr[ps] = f32x4 { 0.f, 0.f, 0.f, 0.f };
                if (R && m < p.M && n_ok)
                    rr[ps] = *reinterpret_cast<const f32x4*>(R + (int64_t)m * p.ldc + n);
            }
        };
        f32x4 wsum4 = { 0.f, 0.f, 0.f, 0.f };
        auto request_epilogue = [&]() {
            if (p.bias && n_ok)
                bias4 = *reinterpret_cast<const f32x4*>(p.bias + n);
            if (LNF && n_ok)
                wsum4 = *reinterpret_cast<const f32x4*>(p.ln_wsum + n);
            request_residual(0);
        };
        // (the split variants hold partial tiles in registers across the exchange below; there the requests wait
        // until the exchange is over)
        if (!SPLIT)
            request_epilogue();
        tile += unit_step;
        const bool more = tile < unit_end;
        if (more) {
            setup(tile, m0, n0, c_off);
            load_tiles(); // in flight while this tile is written out
        }

        if (SPLIT && su_done >= 0) {
            constexpr int TILE_F = BM * BN;
            // contributors of this output tile, its ticket, and where contributor number sp left its partial
            int parts = S, out_tile = sk ? tile_done : su_done / S, g_a = 0;
            const int64_t t0 = (int64_t)tile_done * KT;
            if (sk) {
                g_a = (int)(((t0 + 1) * G + W - 1) / W) - 1; // the workgroup whose stretch holds the tile's first slab
                parts = (int)(((t0 + KT) * G + W - 1) / W) - g_a; // ... up to the one that holds its last slab
            }
            auto slot_of = [&](int sp) -> int64_t {
                if (!sk)
                    return (int64_t)out_tile * S + sp;
                const int gg = g_a + sp;
                return 2 * (int64_t)gg + (gg * W / G > t0 ? 0 : 1);
            };
            float* mine = p.split_ws + (int64_t)su_done * TILE_F + t;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        __hip_atomic_store(mine + ((i * TN + j) * 16 + e) * NT, acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // every lane's partials have left the CU before the ticket is taken
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (t == 0) {
                const int ticket = __hip_atomic_fetch_add(p.split_tickets + out_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const int last = ticket == parts - 1;
                if (last)
                    __hip_atomic_store(p.split_tickets + out_tile, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); // next launch
                last_flag = last;
            }
            __syncthreads();
            const bool is_last = last_flag != 0;
            __syncthreads(); // last_flag is rewritten by the next unit
            if (!is_last) {
                if (!more)
                    break;
                continue;
            }
            // Partials are summed in split order.  The own one comes from the workspace like the others where a second
            // copy of the accumulators would halve the number of resident workgroups (128 x 128 tiles: re-reading it
            // costs a tile of loads); smaller tiles keep it in registers.
            constexpr bool REREAD_OWN = TM * TN >= 4;
            f32x16 own[REREAD_OWN ? 1 : TM][REREAD_OWN ? 1 : TN];
            int my_part = -1;
            if (!REREAD_OWN) {
                my_part = sk ? g_lin - g_a : su_done - out_tile * S;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        own[REREAD_OWN ? 0 : i][REREAD_OWN ? 0 : j] = acc[i][j];
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        acc[i][j][e] = 0.f;
            for (int sp = 0; sp < parts; ++sp) {
                const float* part = p.split_ws + slot_of(sp) * TILE_F + t;
                const bool self = sp == my_part;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            acc[i][j][e] += self ? own[REREAD_OWN ? 0 : i][REREAD_OWN ? 0 : j][e]
                                                 : __hip_atomic_load(part + ((i * TN + j) * 16 + e) * NT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        // one 32x32 block's loads at a time: hoisting all of them would need a register per load
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
        }

        // ---- epilogue: accumulators -> per-wave LDS scratch [32][WTN] -> 16-byte row accesses
        float* scratch = smem + wave * 32 * OSTRIDE;
        if (SPLIT)
            request_epilogue();
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            // the residual rows of a later 32-row band are requested before the accumulators go through LDS, so their
            // latency is covered by the transposition instead of stalling every store
            if (i > 0)
                request_residual(i);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    scratch[(8 * (e >> 2) + 4 * fh + (e & 3)) * OSTRIDE + j * 32 + fr] = acc[i][j][e];
            // the scratch band is private to this wave and a wave's LDS accesses complete in order: no workgroup barrier
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // all rows of the band are finished in registers before the first of them is stored: the wait for the
            // residual loads would otherwise also wait, pass after pass, for the store of the pass before
            f32x4 done[32 / RPS];
#pragma unroll
            for (int ps = 0; ps < 32 / RPS; ++ps) {
                const int row = ps * RPS + srow;
                const f32x4 v = *reinterpret_cast<const f32x4*>(&scratch[row * OSTRIDE + scol]);
                float r[4];
                if (LNF) {
                    const int trow = wm * WTM + i * 32 + row;
                    const float mu = ln_stats[2 * trow], rs = ln_stats[2 * trow + 1];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        r[e] = rs * (v[e] - mu * wsum4[e]) + bias4[e] + rr[ps][e];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        r[e] = v[e] * p.alpha + bias4[e] + rr[ps][e];
                }
                apply_act_block(r, p.act);
                done[ps] = f32x4 { r[0], r[1], r[2], r[3] };
            }
#pragma unroll
            for (int ps = 0; ps < 32 / RPS; ++ps) {
                const int m = em0 + wm * WTM + i * 32 + ps * RPS + srow;
                if (m < p.M && n_ok) {
                    // written through to memory (agent scope) rather than left dirty in this XCD's L2: the next layer's
                    // workgroups run on all XCDs, and what a kernel leaves dirty is written back at its end with nothing
                    // else running (ResNet50 +0.4 %; the non-temporal hint instead: -0.8 %).  A buffer store because that
                    // is the store the compiler lets carry the scope bit: the descriptor starts at the band's first row
                    // (uniform), the lane's offset covers at most 32 rows (ldc < 2^24 on this path).
                    const __amdgpu_buffer_rsrc_t srd_c = __builtin_amdgcn_make_buffer_rsrc(
                        C + (int64_t)(em0 + __builtin_amdgcn_readfirstlane(wm) * WTM + i * 32) * p.ldc, 0, -1, 0x00020000);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, done[ps]), srd_c,
                        (int)((uint32_t)((ps * RPS + srow) * p.ldc + n) * 4u), 0, 16);
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        if (!more)
            break;
        __syncthreads(); // every wave is done with its scratch before the next tile's operands overwrite it
    }
}

// Implicit-GEMM Conv2D and row-major GEMM on fp32 MFMA (v_mfma_f32_32x32x2_f32), gfx950.
//
// One kernel template serves both: the A operand is either a row-major matrix or the
// virtual im2col matrix of an NHWC activation tensor (never materialised: padding is a
// load predicate, the K axis walks (filter row, filter column, input channel) which is a
// contiguous channel run in memory and also the storage order of the converted-JSON
// filters, so weights need no re-layout).  B is always [N][K] with K contiguous.
//
// Tiling: a workgroup of WAVES_M x WAVES_N wave64s owns a BM x BN output tile and walks K
// in slabs of 16.  Global loads are 16-byte per lane into registers, written to LDS rows
// padded to 20 floats (conflict-free 128-bit fragment reads), double-buffered so one
// barrier per slab suffices.  Each lane feeds four consecutive k values from one 128-bit
// LDS read into four MFMAs (the k order inside a slab is permuted identically for A and
// B, which a sum does not notice).  Epilogue: alpha, bias (per column or per row),
// residual add, activation, fused on the accumulators before the only store.
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

#include "common.hpp"
#include "igemm_params.hpp"

namespace fdx {

enum { A_ROWS_VEC = 0, A_CONV_VEC = 1, A_CONV_SCALAR = 2, A_ROWS_SCALAR = 3 };

constexpr int BK = 16;
constexpr int LDS_STRIDE = BK + 4;

template <int BM, int BN, int WAVES_M, int WAVES_N, int A_MODE, int B_VEC>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void igemm_kernel(GemmParams p)
{
    constexpr int NT = 64 * WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int A_LOADS = (BM * 4 + NT - 1) / NT, B_LOADS = (BN * 4 + NT - 1) / NT;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA");
    static_assert(NT % 4 == 0, "loader mapping assumes the k quarter is fixed per thread");

    __shared__ __attribute__((aligned(16))) float As[2][BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN * LDS_STRIDE];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous run of
    // tiles so that tiles sharing an A row block also share that XCD's L2.
    const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
    const int total = tiles_m * tiles_n;
    int id = blockIdx.x;
    {
        const int xcd = id & 7, local = id >> 3, per = total >> 3, rem = total & 7;
        id = xcd * per + (xcd < rem ? xcd : rem) + local;
    }
    const int m0 = (id / tiles_n) * BM, n0 = (id % tiles_n) * BN;

    const int z = blockIdx.z;
    const float* __restrict__ A = p.A + (z / p.inner) * p.a_outer + (z % p.inner) * p.a_inner;
    const float* __restrict__ B = p.B + (z / p.inner) * p.b_outer + (z % p.inner) * p.b_inner;
    const int64_t c_off = (z / p.inner) * p.c_outer + (z % p.inner) * p.c_inner;
    float* __restrict__ C = p.C + c_off;
    const float* __restrict__ R = p.residual ? p.residual + c_off : nullptr;

    const int kq = t & 3; // which 4-float quarter of the 16-wide slab this thread loads

    // ---- per-thread A row state (fixed for the whole K loop)
    bool a_ok[A_LOADS];
    const float* a_ptr[A_LOADS];
    int a_iy0[A_LOADS], a_ix0[A_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int idx = t + i * NT;
        const int m = m0 + (idx >> 2);
        a_ok[i] = (idx < BM * 4) && (m < p.M);
        a_ptr[i] = A;
        a_iy0[i] = a_ix0[i] = 0;
        if (a_ok[i]) {
            if (A_MODE == A_ROWS_VEC || A_MODE == A_ROWS_SCALAR) {
                a_ptr[i] = A + (int64_t)m * p.lda;
            } else {
                const int img = m / (p.OH * p.OW), rem = m - img * (p.OH * p.OW);
                const int oy = rem / p.OW, ox = rem - oy * p.OW;
                a_ptr[i] = A + (int64_t)img * p.H * p.W * p.Cin;
                a_iy0[i] = oy * p.sy - p.pad_top;
                a_ix0[i] = ox * p.sx - p.pad_left;
            }
        }
    }
    // conv k-state of this thread's quarter: input channel, filter column, filter row
    int kc = 0, kfx = 0, kfy = 0;
    if (A_MODE == A_CONV_VEC || A_MODE == A_CONV_SCALAR) {
        const int kk = kq * 4, tap = kk / p.Cin;
        kc = kk - tap * p.Cin;
        kfy = tap / p.kw;
        kfx = tap - kfy * p.kw;
    }
    bool b_ok[B_LOADS];
    const float* b_ptr[B_LOADS];
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int idx = t + i * NT;
        const int n = n0 + (idx >> 2);
        b_ok[i] = (idx < BN * 4) && (n < p.N);
        b_ptr[i] = b_ok[i] ? B + (int64_t)n * p.ldb : B;
    }

    f32x4 ra[A_LOADS], rb[B_LOADS];

    auto load_tiles = [&](int kt) {
        const int k = kt * BK + kq * 4;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            f32x4 v = { 0.f, 0.f, 0.f, 0.f };
            if (A_MODE == A_ROWS_VEC) {
                if (a_ok[i] && k < p.K)
                    v = *reinterpret_cast<const f32x4*>(a_ptr[i] + k);
            } else if (A_MODE == A_ROWS_SCALAR) {
                if (a_ok[i]) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (k + j < p.K)
                            v[j] = a_ptr[i][k + j];
                }
            } else if (A_MODE == A_CONV_VEC) {
                const int iy = a_iy0[i] + kfy * p.dy, ix = a_ix0[i] + kfx * p.dx;
                if (a_ok[i] && kfy < p.kh && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W)
                    v = *reinterpret_cast<const f32x4*>(a_ptr[i] + ((int64_t)(iy * p.W + ix) * p.Cin + kc));
            } else {
                // the quarter's four k values one by one, (channel, filter column, filter row) carried along instead of
                // divided out of k for every element (two integer divisions per loaded float made the 3-channel stem
                // convolutions instruction-bound); k < K is the same as filter row < kh
                if (a_ok[i]) {
                    int c = kc, fx = kfx, fy = kfy;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (fy < p.kh) {
                            const int iy = a_iy0[i] + fy * p.dy, ix = a_ix0[i] + fx * p.dx;
                            if (iy >= 0 && iy < p.H && ix >= 0 && ix < p.W)
                                v[j] = a_ptr[i][(int64_t)(iy * p.W + ix) * p.Cin + c];
                        }
                        if (++c == p.Cin) {
                            c = 0;
                            if (++fx == p.kw) {
                                fx = 0;
                                ++fy;
                            }
                        }
                    }
                }
            }
            ra[i] = v;
        }
        if (A_MODE == A_CONV_VEC || A_MODE == A_CONV_SCALAR) { // advance the quarter's (fy, fx, c) by one slab
            kc += BK;
            while (kc >= p.Cin) {
                kc -= p.Cin;
                if (++kfx == p.kw) {
                    kfx = 0;
                    ++kfy;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            f32x4 v = { 0.f, 0.f, 0.f, 0.f };
            if (B_VEC) {
                if (b_ok[i] && k < p.K)
                    v = *reinterpret_cast<const f32x4*>(b_ptr[i] + k);
            } else if (b_ok[i]) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (k + j < p.K)
                        v[j] = b_ptr[i][k + j];
            }
            rb[i] = v;
        }
    };
    auto store_tiles = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const int idx = t + i * NT;
            if (idx < BM * 4)
                *reinterpret_cast<f32x4*>(&As[buf][(idx >> 2) * LDS_STRIDE + kq * 4]) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const int idx = t + i * NT;
            if (idx < BN * 4)
                *reinterpret_cast<f32x4*>(&Bs[buf][(idx >> 2) * LDS_STRIDE + kq * 4]) = rb[i];
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e)
                acc[i][j][e] = 0.f;

    const int KT = (p.K + BK - 1) / BK;
    const int fr = lane & 31, fh = lane >> 5;

    load_tiles(0);
    store_tiles(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < KT)
            load_tiles(kt + 1);
#pragma unroll
        for (int k8 = 0; k8 < BK / 8; ++k8) {
            f32x4 af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                af[i] = *reinterpret_cast<const f32x4*>(
                    &As[buf][(wm * WTM + i * 32 + fr) * LDS_STRIDE + k8 * 8 + fh * 4]);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                bf[j] = *reinterpret_cast<const f32x4*>(
                    &Bs[buf][(wn * WTN + j * 32 + fr) * LDS_STRIDE + k8 * 8 + fh * 4]);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][e], bf[j][e], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < KT)
            store_tiles(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue.  32x32 accumulator layout: element e of lane l is
    // row 8*(e/4) + 4*(l/32) + e%4, column l%32.
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * WTN + j * 32 + fr;
        if (n >= p.N)
            continue;
        const float bcol = (p.bias && !p.bias_per_row) ? p.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            float r[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (e >> 2) + 4 * fh + (e & 3);
                r[e] = acc[i][j][e] * p.alpha + bcol;
                if (m < p.M) {
                    if (p.bias && p.bias_per_row)
                        r[e] += p.bias[m];
                    if (R)
                        r[e] += R[(int64_t)m * p.ldc + n];
                }
            }
            apply_act_block(r, p.act);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + wm * WTM + i * 32 + 8 * (e >> 2) + 4 * fh + (e & 3);
                if (m < p.M)
                    C[(int64_t)m * p.ldc + n] = r[e];
            }
        }
    }
}


#include "igemm_fast.hpp"

// ------------------------------------------------------------------ dispatch

static int g_forced_tile = -1; // tests force a tile configuration through fdx_debug_force_tile
static bool g_dual_one_launch = true; // tests run a two-input convolution as two launches through fdx_debug_dual_conv

template <int BM, int BN, int WM, int WN>
static void launch_cfg(const GemmParams& p, int a_mode, int b_vec, int batch, hipStream_t s)
{
    const int tiles = ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
    dim3 grid(tiles, 1, batch), block(64 * WM * WN);
#define FDX_IGEMM_CASE(AM, BV)                                                              \
    if (a_mode == AM && b_vec == BV) {                                                      \
        hipLaunchKernelGGL((igemm_kernel<BM, BN, WM, WN, AM, BV>), grid, block, 0, s, p);   \
        return;                                                                             \
    }
    FDX_IGEMM_CASE(A_ROWS_VEC, 1)
    FDX_IGEMM_CASE(A_ROWS_VEC, 0)
    FDX_IGEMM_CASE(A_CONV_VEC, 1)
    FDX_IGEMM_CASE(A_CONV_VEC, 0)
    FDX_IGEMM_CASE(A_CONV_SCALAR, 1)
    FDX_IGEMM_CASE(A_CONV_SCALAR, 0)
    FDX_IGEMM_CASE(A_ROWS_SCALAR, 1)
    FDX_IGEMM_CASE(A_ROWS_SCALAR, 0)
#undef FDX_IGEMM_CASE
}

// Persistent launch: as many workgroups as fit on the chip at once (occupancy x CUs, cached per
// kernel), or one per tile when there are fewer tiles than that.
static int g_persist_scale = 0; // 0 = resident workgroups; tests and tuning may override the grid cap
template <typename K>
static int resident_workgroups(K kernel, int threads)
{
    // keyed by the kernel's address: every instantiation has the same function type, so a static inside this template
    // would be one value for all of them (callers hold g_igemm_mutex)
    static std::map<const void*, int> cache;
    int& resident = cache[reinterpret_cast<const void*>(kernel)];
    if (resident == 0) {
        int per_cu = 1, dev = 0;
        hipDeviceProp_t prop;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess || per_cu < 1)
            per_cu = 1;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess)
            prop.multiProcessorCount = 256;
        resident = per_cu * prop.multiProcessorCount;
    }
    return resident;
}

// Strip width (in column tiles) for a whole-tile launch of `grid` workgroups, from a model of what the eight L2s fetch:
// with `ns` strips every strip reads all of A once (A x ns in total) and each XCD reads its strip's share of B, once if
// that share stays in its L2 between rounds of workgroups and once per round otherwise.
static int g_strips = -1; // FDX_STRIPS=0 keeps the row-by-row order
static int g_forced_strips = 0; // fdx_debug_force_strips
static int pick_strip_width(const GemmParams& q, int bm, int bn, int grid)
{
    if (g_strips < 0) {
        const char* e = std::getenv("FDX_STRIPS");
        g_strips = (e && e[0] == '0') ? 0 : 1;
    }
    if (q.batch != 1)
        return 0;
    const int tiles_m = (q.M + bm - 1) / bm, tiles_n = (q.N + bn - 1) / bn;
    if (g_forced_strips > 0) // test hook: this many strips wherever there are as many column tiles
        return g_forced_strips <= tiles_n ? (tiles_n + g_forced_strips - 1) / g_forced_strips : 0;
    if (!g_strips)
        return 0;
    const double a_bytes = 4.0 * q.M * q.K, b_bytes = 4.0 * q.N * q.K;
    const int rounds = (tiles_m * tiles_n + grid - 1) / grid;
    int best_ns = 1;
    double best_cost = 0.0;
    for (int ns = 1; ns <= 8 && ns <= tiles_n; ns *= 2) {
        const double share = b_bytes / ns;
        const double cost = a_bytes * ns + 8.0 * share * (share <= 2.0e6 ? 1 : rounds);
        if (ns == 1 || cost < 0.9 * best_cost) { // a change of order has to promise a tenth less traffic
            best_cost = cost;
            best_ns = ns;
        }
    }
    return best_ns == 1 ? 0 : (tiles_n + best_ns - 1) / best_ns;
}

template <typename K>
static void launch_persistent(K kernel, int tiles, const GemmParams& q, hipStream_t s, int threads = 256, int bm = 0, int bn = 0)
{
    const int resident = resident_workgroups(kernel, threads);
    const int cap = g_persist_scale > 0 ? g_persist_scale : resident;
    const int grid = tiles < cap ? tiles : cap;
    GemmParams r = q;
    r.strip_w = bm > 0 ? pick_strip_width(q, bm, bn, grid) : 0;
    hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3((unsigned)threads), 0, s, r);
}

#include "pw_stream.hpp"

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// library-owned scratch of the split-K variant: partial tiles and one ticket per output tile
// (tickets are zero between launches: the last unit of a tile resets its ticket)
static float* g_split_ws = nullptr;
static int* g_split_tickets = nullptr;
constexpr size_t kSplitWsBytes = 192u << 20;
constexpr int kSplitTickets = 1 << 16;

static bool split_prepare()
{
    if (g_split_ws && g_split_tickets)
        return true;
    if (hipMalloc(&g_split_ws, kSplitWsBytes) != hipSuccess)
        return false;
    if (hipMalloc(&g_split_tickets, sizeof(int) * kSplitTickets) != hipSuccess
        || zero_device(g_split_tickets, sizeof(int) * kSplitTickets) != hipSuccess)
        return false;
    return true;
}

static void tile_of(int cfg, int& bm, int& bn, int& bk)
{
    switch (cfg) {
    case 10: bm = 128; bn = 128; bk = 16; break;
    case 11: bm = 128; bn = 64; bk = 16; break;
    case 12: bm = 64; bn = 64; bk = 16; break;
    case 13: bm = 128; bn = 128; bk = 32; break;
    case 14: bm = 128; bn = 64; bk = 32; break;
    case 15: bm = 64; bn = 64; bk = 32; break;
    case 16: bm = 128; bn = 128; bk = 32; break;
    case 17: bm = 128; bn = 128; bk = 32; break;
    case 18: bm = 256; bn = 128; bk = 32; break;
    default: bm = 64; bn = 64; bk = 32; break;
    }
}

// whether `splits` K ranges per tile are possible for `split_tiles` tiles of this configuration: enough slabs per
// range, and the partial tiles and tickets fit the scratch
static bool split_fits(int cfg, int splits, int64_t split_tiles, const GemmParams& q)
{
    int bm, bn, bk;
    tile_of(cfg, bm, bn, bk);
    return splits >= 2 && q.K / bk >= 2 * splits && split_tiles <= kSplitTickets
        && (size_t)split_tiles * splits * bm * bn * sizeof(float) <= kSplitWsBytes && split_tiles * splits < (1 << 30);
}

// One launch of the split variant.  hybrid: the tiles that fill whole rounds of resident workgroups are computed
// whole and only the last, partial round is cut into K ranges, so that every workgroup ends at about the same time;
// otherwise every tile is cut.  Returns false when the cut does not fit the scratch.
// mode 2 (stream-K, splits == 0): one workgroup per resident slot, each with an equal stretch of the slabs of all tiles;
// needs two workspace slots per workgroup and a ticket per tile.
template <typename K>
static bool launch_split(K kernel, int tiles, int splits, int mode, int cfg, GemmParams& q, hipStream_t s)
{
    const int resident = g_persist_scale > 0 ? g_persist_scale : resident_workgroups(kernel, 256);
    if (mode == 2) {
        int bm, bn, bk;
        tile_of(cfg, bm, bn, bk);
        const int64_t slabs = (int64_t)tiles * (q.K / bk);
        const int grid = (int)std::min<int64_t>(resident, slabs);
        if (tiles > kSplitTickets || (size_t)grid * 2 * bm * bn * sizeof(float) > kSplitWsBytes || slabs >= (1LL << 40))
            return false;
        q.splits = 0;
        q.split_dp_tiles = 0;
        hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(256), 0, s, q);
        return true;
    }
    const bool hybrid = mode == 1;
    const int dp = hybrid ? (tiles / resident) * resident : 0;
    if (tiles - dp > 0 && !split_fits(cfg, splits, tiles - dp, q))
        return false;
    q.split_dp_tiles = dp;
    launch_persistent(kernel, dp + (tiles - dp) * splits, q, s);
    return true;
}

static bool launch_fast(int cfg, int splits, int mode, const GemmParams& q0, bool conv, int batch, hipStream_t s)
{
    GemmParams q = q0;
    q.splits = splits;
    q.split_dp_tiles = 0;
    q.split_ws = g_split_ws;
    q.split_tickets = g_split_tickets;
    q.strip_w = 0; // set per whole-tile launch

    bool ok = true;
#define FDX_FAST(BM_, BN_, BK_)                                                                                  \
    {                                                                                                            \
        const int tiles = ((q.M + BM_ - 1) / BM_) * ((q.N + BN_ - 1) / BN_) * batch;                             \
        if (mode == 2) {                                                                                         \
            if (conv)                                                                                            \
                ok = launch_split(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, true, true, true>, tiles, splits, mode, cfg, q, s); \
            else                                                                                                 \
                ok = launch_split(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, false, true, true>, tiles, splits, mode, cfg, q, s); \
        } else if (splits > 1) {                                                                                 \
            if (conv)                                                                                            \
                ok = launch_split(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, true, true>, tiles, splits, mode, cfg, q, s); \
            else                                                                                                 \
                ok = launch_split(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, false, true>, tiles, splits, mode, cfg, q, s); \
        } else if (conv)                                                                                         \
            launch_persistent(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, true>, tiles, q, s, 256, BM_, BN_);         \
        else if (q.A2)                                                                                           \
            launch_persistent(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, false, false, false, true>, tiles, q, s, 256, BM_, BN_); \
        else                                                                                                     \
            launch_persistent(igemm_fast_kernel<BM_, BN_, 2, 2, BK_, false>, tiles, q, s, 256, BM_, BN_);        \
    }
        // eight-wave variants: more waves per SIMD to cover LDS and global latency, or a 256-row tile that halves the
        // operand traffic per FLOP
#define FDX_FAST8(BM_, BN_, WM_, WN_)                                                                            \
    {                                                                                                            \
        const int tiles = ((q.M + BM_ - 1) / BM_) * ((q.N + BN_ - 1) / BN_) * batch;                             \
        if (conv)                                                                                                \
            launch_persistent(igemm_fast_kernel<BM_, BN_, WM_, WN_, 32, true>, tiles, q, s, 512, BM_, BN_);      \
        else                                                                                                     \
            launch_persistent(igemm_fast_kernel<BM_, BN_, WM_, WN_, 32, false>, tiles, q, s, 512, BM_, BN_);     \
    }
    if (q.ln_wsum) { // rows normalised on the way: whole tiles of the 32-float slab configurations
        switch (cfg) {
        case 13: launch_persistent(igemm_fast_kernel<128, 128, 2, 2, 32, false, false, false, false, true>,
            ((q.M + 127) / 128) * ((q.N + 127) / 128) * batch, q, s, 256, 128, 128); break;
        case 14: launch_persistent(igemm_fast_kernel<128, 64, 2, 2, 32, false, false, false, false, true>,
            ((q.M + 127) / 128) * ((q.N + 63) / 64) * batch, q, s, 256, 128, 64); break;
        default: launch_persistent(igemm_fast_kernel<64, 64, 2, 2, 32, false, false, false, false, true>,
            ((q.M + 63) / 64) * ((q.N + 63) / 64) * batch, q, s, 256, 64, 64); break;
        }
        return true;
    }
        switch (cfg) {
        case 10: FDX_FAST(128, 128, 16) break;
        case 11: FDX_FAST(128, 64, 16) break;
        case 12: FDX_FAST(64, 64, 16) break;
        case 13: FDX_FAST(128, 128, 32) break;
        case 14: FDX_FAST(128, 64, 32) break;
        case 16: FDX_FAST8(128, 128, 2, 4) break;
        case 17: FDX_FAST8(128, 128, 4, 2) break;
        case 18: FDX_FAST8(256, 128, 4, 2) break;
        default: FDX_FAST(64, 64, 32) break;
        }
#undef FDX_FAST
#undef FDX_FAST8
    return ok;
}

// First sight of a problem shape on the fast path: time every tile configuration once on the
// real operands (the launches are idempotent) and remember the winner.  Tile count versus
// resident workgroups, K depth and output width interact too irregularly for a closed rule.
// A choice is (configuration, K splits, mode) packed as cfg + 100 * splits + 10000 * mode, mode 0 = every tile cut into
// `splits` K ranges, 1 = hybrid (only the last partial round is cut), 2 = stream-K (splits unused).  Cutting every tile
// is tried only where a configuration has few tiles for the chip; the hybrid cut of the last partial round wherever
// there is one.
// (TuneKey: igemm_params.hpp; conv = 2 rows hold the one-launch / two-launch choice of a depthwise + 1x1 pair)
static std::map<TuneKey, int> g_tuned;
static std::mutex g_tune_mutex; // the table only; never held across a launch
static bool g_tune_frozen = false;

bool tune_lookup(const TuneKey& key, int* choice)
{
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    auto it = g_tuned.find(key);
    if (it == g_tuned.end())
        return false;
    *choice = it->second;
    return true;
}
void tune_store(const TuneKey& key, int choice)
{
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    g_tuned[key] = choice;
}
static std::chrono::steady_clock::time_point g_tune_end; // end of the last timing run (epoch = none yet)
static std::mutex g_tune_end_mutex;
void tune_mark()
{
    std::lock_guard<std::mutex> lock(g_tune_end_mutex);
    g_tune_end = std::chrono::steady_clock::now();
}
void tune_settle_clock(const std::function<bool()>& launch)
{
    using namespace std::chrono;
    {
        std::lock_guard<std::mutex> lock(g_tune_end_mutex);
        if (steady_clock::now() - g_tune_end < milliseconds(5))
            return;
    }
    const auto t0 = steady_clock::now();
    bool ok = true;
    while (ok && steady_clock::now() - t0 < milliseconds(30)) {
        for (int r = 0; r < 3 && ok; ++r)
            ok = launch();
        if (hipStreamSynchronize(stream()) != hipSuccess)
            break;
    }
    tune_mark();
}

// Whether first sights of a shape may be timed.  Off unless the caller asks (fdx_tuner_timing(1) or FDX_AUTOTUNE=1 in
// the environment): a timing run launches a few thousand candidates, about a second for a ResNet50 at batch 64, which a
// drop-in predict must not spend on its first call.  With timing off every choice (tile, K cut, direct against Winograd,
// block forms) follows the closed rules, the same in every process.
static int g_tune_timing = -1; // -1 = not read yet; guarded by g_tune_mutex
static bool tune_timing_locked()
{
    if (g_tune_timing < 0) {
        const char* e = std::getenv("FDX_AUTOTUNE");
        g_tune_timing = (e && e[0] == '1') ? 1 : 0;
    }
    return g_tune_timing == 1;
}
bool tune_frozen()
{
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    return g_tune_frozen || !tune_timing_locked();
}
static int g_split_enabled = 1; // FDX_SPLITK=0 keeps the tuner to one K range per tile

// general_cfg >= 0: the general kernel's configuration for this shape competes too (narrow outputs, where half of a
// 64-wide fast tile is idle); general_launch runs it once on the caller's unshifted parameters
// stream_ok: the row-streaming short-K kernel (configuration 30, pw_stream.hpp) competes as well
constexpr int kStreamCfg = 30;
template <typename F, typename G>
static int autotune(const GemmParams& q, bool conv, int batch, int unit, hipStream_t s, int general_cfg, F general_launch,
    bool stream_ok, G stream_launch)
{
    static const bool split_env = [] { const char* sp = std::getenv("FDX_SPLITK"); return !(sp && sp[0] == '0'); }();
    g_split_enabled = split_env ? 1 : 0;
    TuneKey key;
    std::memset(&key, 0, sizeof key);
    key.conv = conv; key.M = q.M; key.N = q.N; key.K = q.K; key.Cin = conv ? q.Cin : 0; key.kh = conv ? q.kh : 0;
    key.kw = conv ? q.kw : 0; key.sy = conv ? q.sy : 0; key.sx = conv ? q.sx : 0; key.batch = batch; key.res = q.residual != nullptr;
    int known = -1;
    if (tune_lookup(key, &known))
        return known;
    if (tune_frozen())
        return -1; // an unseen shape under a frozen table takes the closed rule of run_igemm: no timing, same choice every run
    hipEvent_t a, b;
    if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess)
        return -1;
    int best = -1, best_split = -1;
    float best_ms = 1e30f, best_split_ms = 1e30f;
    const bool can_split = g_split_enabled && split_prepare();
    // three launches back to back, the faster of two such rounds: candidates within a percent of each other are
    // common, and a single round of a 30 us kernel is too short a window to tell them apart
    auto timed = [&](auto&& launch) -> float {
        float best_round = 1e30f;
        for (int round = 0; round < 2; ++round) {
            (void)hipEventRecord(a, s);
            for (int r = 0; r < 3; ++r)
                launch();
            (void)hipEventRecord(b, s);
            float ms = 1e30f;
            if (hipEventSynchronize(b) == hipSuccess && hipEventElapsedTime(&ms, a, b) == hipSuccess && ms < best_round)
                best_round = ms;
        }
        return best_round;
    };
    bool clock_settled = false;
    for (int cfg = 10; cfg <= 18; ++cfg) {
        if (cfg >= 13 && unit % 32 != 0)
            continue;
        int bm, bn, bk;
        tile_of(cfg, bm, bn, bk);
        const int64_t tiles = (int64_t)((q.M + bm - 1) / bm) * ((q.N + bn - 1) / bn) * batch;
        if (bn > 64 && q.N <= bn / 2)
            continue; // a tile at least twice as wide as the output only idles half of every MFMA
        static const int kChoices[][2] = { { 1, 0 }, { 2, 0 }, { 3, 0 }, { 4, 0 }, { 2, 1 }, { 3, 1 }, { 4, 1 }, { 6, 1 }, { 8, 1 }, { 0, 2 } };
        for (const auto& ch : kChoices) {
            const int splits = ch[0], mode = ch[1];
            const bool hybrid = mode == 1;
            if (splits != 1 && !(can_split && cfg <= 15))
                continue;
            static const bool streamk_on = [] { const char* e = std::getenv("FDX_STREAMK"); return !(e && e[0] == '0'); }();
            if (mode == 2 && !streamk_on)
                continue;
            if (splits > 1 && mode == 0 && !(tiles <= 1024 && split_fits(cfg, splits, tiles, q)))
                continue;
            if (hybrid && tiles > 16384)
                continue;
            if (!launch_fast(cfg, splits, mode, q, conv, batch, s)) // warm-up; false = the cut does not fit
                continue;
            if (!clock_settled) {
                tune_settle_clock([&] { return launch_fast(cfg, splits, mode, q, conv, batch, s); });
                clock_settled = true;
            }
            const float ms = timed([&] { launch_fast(cfg, splits, mode, q, conv, batch, s); });
            if (splits == 1) {
                if (ms < best_ms) {
                    best_ms = ms;
                    best = cfg;
                }
            } else {
                // What a cut costs beyond its own time: partial tiles written and read back (K ranges, and the last
                // round of the hybrid form), and in the stream-K form every tile's operands fetched at a K phase of
                // its own, so that tiles of one row block no longer share them in L2 (measured on ResNet50's
                // 14 x 14 and 7 x 7 1x1 layers: 3.7 times the algorithmic bytes).  A cut has to win by more than that
                // handicap to be taken: 4 % of its time for K ranges, 15 % for stream-K (which wins by 9 % on those 1x1
                // layers, by 15-20 % on deep 3x3 convolutions and by more on a Dense with few rows).
                const float score = ms * (mode == 2 ? 1.15f : 1.04f);
                if (score < best_split_ms) {
                    best_split_ms = score;
                    best_split = cfg + 100 * splits + 10000 * mode;
                }
            }
        }
    }
    if (general_cfg >= 0) {
        general_launch();
        const float ms = timed(general_launch);
        if (ms < best_ms) {
            best_ms = ms;
            best = general_cfg;
        }
    }
    if (stream_ok) {
        stream_launch();
        const float ms = timed(stream_launch);
        if (ms < best_ms) {
            best_ms = ms;
            best = kStreamCfg;
        }
    }
    (void)hipEventDestroy(a);
    (void)hipEventDestroy(b);
    tune_mark();
    static const bool log_picks = [] { const char* e = std::getenv("FDX_TUNE_LOG"); return e && e[0] == '1'; }();
    if (log_picks)
        std::fprintf(stderr, "[fdx tune] conv=%d M=%d N=%d K=%d Cin=%d k=%dx%d s=%d res=%d: plain %d %.1f us, split %d %.1f us with its handicap\n", (int)conv,
            q.M, q.N, q.K, q.Cin, q.kh, q.kw, q.sy, (int)(q.residual != nullptr), best, best_ms * 1e3f / 3, best_split, best_split_ms * 1e3f / 3);
    if (best_split >= 0 && (best < 0 || best_split_ms < best_ms))
        best = best_split;
    if (log_picks)
        std::fprintf(stderr, "[fdx tune]   -> %d\n", best);
    tune_store(key, best);
    return best;
}

// the tuner's table and its timing runs, and the order in which launches that share the split workspace reach the
// stream, are per process: host threads take turns here
static std::mutex g_igemm_mutex;

static fdx_status run_igemm(GemmParams& p, bool conv, int batch, const char* family, double algorithmic_flops = 0.0)
{
    std::lock_guard<std::mutex> lock(g_igemm_mutex);
    int a_mode;
    if (conv)
        a_mode = (p.Cin % 4 == 0 && aligned16(p.A)) ? A_CONV_VEC : A_CONV_SCALAR;
    else
        a_mode = (p.K % 4 == 0 && p.lda % 4 == 0 && aligned16(p.A) && p.a_outer % 4 == 0 && p.a_inner % 4 == 0)
            ? A_ROWS_VEC
            : A_ROWS_SCALAR;
    const int b_vec = (p.K % 4 == 0 && p.ldb % 4 == 0 && aligned16(p.B) && p.b_outer % 4 == 0 && p.b_inner % 4 == 0) ? 1 : 0;

    auto blocks = [&](int bm, int bn) { return (int64_t)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * batch; };
    hipStream_t s = stream();

    // ---- fast path eligibility (see igemm_fast_kernel)
    const bool out_ok = p.N % 4 == 0 && p.ldc % 4 == 0 && aligned16(p.C) && p.c_outer % 4 == 0 && p.c_inner % 4 == 0
        && (!p.residual || aligned16(p.residual)) && (!p.bias || aligned16(p.bias)) && !p.bias_per_row;
    const int64_t b_bytes = ((int64_t)(p.N - 1) * p.ldb + p.K) * 4;
    int64_t a_bytes, a_shift = 0;
    bool a_ok;
    if (p.pix_stride == 0)
        p.pix_stride = p.Cin;
    if (conv) {
        a_shift = ((int64_t)p.pad_top * p.W + p.pad_left) * p.pix_stride;
        a_bytes = ((int64_t)(p.M / (p.OH * p.OW)) * p.H * p.W * p.pix_stride + a_shift) * 4 + 64;
        a_ok = a_mode == A_CONV_VEC && p.Cin % 16 == 0 && p.kh * p.kw <= 64;
    } else {
        a_bytes = ((int64_t)(p.M - 1) * p.lda + (p.a_valid_k > 0 ? p.a_valid_k : p.K)) * 4;
        a_ok = a_mode == A_ROWS_VEC && p.K % 16 == 0;
    }
    const bool fast_ok = out_ok && a_ok && b_vec && a_bytes < (1LL << 31) && b_bytes < (1LL << 31) && p.ldc < (1LL << 24);
    const int unit = conv ? p.Cin : p.K;

    int cfg = g_forced_tile, splits = 1, mode = 0;
    auto unpack = [&]() { // configuration + 100 * splits + 10000 * mode
        mode = cfg / 10000;
        splits = mode == 2 ? 0 : std::max(1, (cfg % 10000) / 100);
        cfg %= 100;
    };
    const bool stream_ok = pw_stream_ok(p, conv, batch, a_bytes, b_bytes) && b_vec;
    // A choice comes from a test hook, from this process's timing runs, or from an imported table: whatever its source, it
    // is only taken where this problem meets the kernel's conditions, and a split choice only with the workspace in
    // place (a process that imports its table has not timed anything, so nothing else would have allocated it).
    auto settle = [&]() {
        if (cfg >= 100)
            unpack();
        if (cfg == kStreamCfg && !stream_ok)
            cfg = -1;
        if (cfg >= 10 && cfg != kStreamCfg && (!fast_ok || (cfg >= 13 && unit % 32 != 0)))
            cfg = -1;
        if (cfg < 10 || mode > 2 || mode < 0 || splits < 0 || splits > 64 || cfg == kStreamCfg) {
            splits = 1;
            mode = 0;
        }
        if (cfg >= 10 && splits != 1 && (cfg > 15 || !split_prepare())) {
            splits = 1;
            mode = 0;
        }
    };
    settle();
    auto launch_general = [&](int c) {
        switch (c) {
        case 0: launch_cfg<128, 128, 2, 2>(p, a_mode, b_vec, batch, s); break;
        case 1: launch_cfg<128, 64, 2, 2>(p, a_mode, b_vec, batch, s); break;
        case 2: launch_cfg<128, 32, 4, 1>(p, a_mode, b_vec, batch, s); break;
        default: launch_cfg<64, 64, 2, 2>(p, a_mode, b_vec, batch, s); break;
        }
    };
    if (p.ln_wsum) {
        // rows normalised on the way: whole tiles, 32-float slab, nothing timed
        const bool ln_ok = !conv && batch == 1 && fast_ok && p.a_valid_k == 0 && !p.A2 && p.K % 32 == 0 && p.alpha == 1.f && aligned16(p.ln_wsum);
        if (!ln_ok) {
            set_error("igemm: this normalising problem needs the fast path");
            return FDX_ERR_UNSUPPORTED;
        }
        if (cfg < 13 || cfg > 15)
            cfg = -1;
        splits = 1;
        mode = 0;
        if (cfg < 0)
            cfg = (p.K >= 1024 && p.N % 128 == 0 && blocks(128, 128) >= 2048) ? 13 : 15;
    } else if (p.A2) {
        // two-source rows: whole tiles of the four-wave fast kernel only, nothing timed
        const int64_t a2_bytes = (int64_t)(p.OH > 0 && p.OW > 0 ? p.M / (p.OH * p.OW) : 0) * p.H2 * p.W2 * p.C2 * 4;
        const bool dual_ok = !conv && batch == 1 && fast_ok && p.a_valid_k == 0 && aligned16(p.A2) && p.C2 % 4 == 0 && p.K1 > 0
            && p.K1 % 16 == 0 && p.K > p.K1 && (p.K - p.K1) % 16 == 0 && p.K - p.K1 <= p.C2 && a2_bytes > 0 && a2_bytes < (1LL << 31)
            && p.s2y > 0 && p.s2x > 0 && (int64_t)(p.OH - 1) * p.s2y < p.H2 && (int64_t)(p.OW - 1) * p.s2x < p.W2
            && p.M == (p.M / (p.OH * p.OW)) * p.OH * p.OW;
        if (!dual_ok) {
            set_error("igemm: this two-source problem needs the fast path");
            return FDX_ERR_UNSUPPORTED;
        }
        p.a2_records = (uint32_t)a2_bytes;
        const bool slab32 = p.K % 32 == 0 && p.K1 % 32 == 0;
        if (cfg < 10 || cfg > 15 || (cfg >= 13 && !slab32))
            cfg = -1;
        splits = 1;
        mode = 0;
        if (cfg < 0) {
            if (p.K >= 1024 && p.N % 128 == 0 && blocks(128, 128) >= 2048)
                cfg = slab32 ? 13 : 10;
            else
                cfg = (slab32 && p.K >= 128) ? 15 : 12;
        }
    } else if (cfg < 0) {
        if (fast_ok && p.N >= 16 && 2.0 * p.M * (double)p.N * p.K * batch >= 2e8) {
            GemmParams q = p;
            q.A = p.A - a_shift;
            q.a_records = (uint32_t)a_bytes;
            q.b_records = (uint32_t)b_bytes;
            q.batch = batch;
            // below 64 output columns the general kernel's narrow tile is a candidate of its own, unless only the
            // fast path can read this operand
            const bool general_ok = p.N < 64 && p.a_valid_k == 0 && !(conv && p.pix_stride != p.Cin);
            const int general_cfg = !general_ok ? -1 : p.N <= 32 ? 2 : (blocks(128, 64) >= 512 ? 1 : 3);
            cfg = autotune(q, conv, batch, unit, s, general_cfg, [&] { launch_general(general_cfg); }, stream_ok,
                [&] { pw_stream_launch(p, a_bytes, b_bytes, s); });
            settle();
        }
        static const bool closed_cuts = [] { const char* e = std::getenv("FDX_CLOSED_SPLIT"); return !(e && e[0] == '0'); }();
        if (cfg >= 0) {
        } else if (stream_ok && p.K <= 32 && p.N <= 160 && p.M >= 65536) {
            // very short rows over a long map (MobileNetV2's first expansions): the row-streaming kernel
            cfg = kStreamCfg;
        } else if (fast_ok && p.N >= 64) {
            // what the timing runs pick most often: the 64 x 64 tile at four or five workgroups per CU, with the
            // 32-float slab where K is long enough for it; the 128 x 128 tile only for problems that are large in
            // every dimension; the 128 x 64 tile with the short slab for wide outputs from short rows, where the
            // stores dominate
            if (p.K >= 1024 && p.N % 128 == 0 && blocks(128, 128) >= 2048)
                cfg = unit % 32 == 0 ? 13 : 10;
            else if (p.K <= 96 && p.N >= 128 && blocks(128, 64) >= 1024)
                cfg = 11;
            else
                cfg = (unit % 32 == 0 && p.K >= 128) ? 15 : 12;
            // Fewer 64 x 64 tiles than one round of resident workgroups (four per CU) and a long K: the chip is filled
            // by cutting K instead.  Below one tile per CU every tile is cut into equal K ranges, about two workgroups
            // per CU in total (a Dense with few rows: 2.8 times faster at 64 x 1000 x 2048); from there up to one
            // round the stream-K form spreads the slabs of all tiles evenly over the resident workgroups (10-12 %
            // faster on ResNet50's 14 x 14 and 7 x 7 1x1 layers).  Both forms add their partial tiles in a fixed order.
            if (closed_cuts && (cfg == 15 || cfg == 12)) {
                const int64_t t64 = blocks(64, 64);
                const int slabs = p.K / (cfg == 15 ? 32 : 16);
                if (t64 < 256 && p.K >= 512) {
                    int want = (int)std::min<int64_t>(8, (512 + t64 - 1) / t64);
                    while (want >= 2 && slabs < 4 * want)
                        --want;
                    if (want >= 2) {
                        splits = want;
                        mode = 0;
                    }
                } else if (t64 < 1024 && p.K >= 1024 && cfg == 15) {
                    splits = 0;
                    mode = 2;
                }
                if (splits != 1)
                    settle(); // the cut needs its workspace
            }
        } else if (p.N <= 32)
            cfg = 2;
        else if (p.N <= 64)
            cfg = blocks(128, 64) >= 512 ? 1 : 3;
        else if (blocks(128, 128) >= 512)
            cfg = 0;
        else if (blocks(128, 64) >= 512)
            cfg = 1;
        else
            cfg = 3;
    }

    if (cfg < 10 && p.a_valid_k > 0) { // only the buffer loads of the fast path stop at the real extent
        set_error("igemm: rows shorter than K need the fast path");
        return FDX_ERR_UNSUPPORTED;
    }
    if (cfg < 10 && conv && p.pix_stride != p.Cin) {
        set_error("igemm: a strided-pixel view needs the fast path");
        return FDX_ERR_INVALID;
    }
    profile_begin();
    if (cfg == kStreamCfg) {
        pw_stream_launch(p, a_bytes, b_bytes, s);
    } else if (cfg >= 10) {
        GemmParams q = p;
        q.A = p.A - a_shift;
        q.a_records = (uint32_t)a_bytes;
        q.b_records = (uint32_t)b_bytes;
        q.batch = batch;
        if (!launch_fast(cfg, splits, mode, q, conv, batch, s))
            launch_fast(cfg, 1, 0, q, conv, batch, s); // the requested cut does not fit the scratch
    } else {
        launch_general(cfg);
    }
    const double flops = algorithmic_flops > 0.0 ? algorithmic_flops : 2.0 * p.M * (double)p.N * p.K * batch;
    profile_end(family, flops, 0.0);
    FDX_LAUNCH_CHECK();
    return FDX_OK;
}

// ------------------------------------------------------------------ stem convolutions (few input channels, stride 2)
// A k x k stride-2 convolution over c <= 4 channels is a (k'/2) x (k'/2) stride-1 convolution over the 2x2
// space-to-depth image with 4c channels (k' = k rounded up to even, the extra filter row / column zero).  In that view
// one filter row reads k'/2 neighbouring pixels = one contiguous run of 2 k' c floats, which the fast path walks as
// Cin = run, kw = 1 with a pixel pitch of 4c floats -- instead of gathering c floats per tap through scalar loads.
// one thread per (space-to-depth pixel, source row): 2c contiguous input floats become 2c contiguous output floats
__global__ void s2d_kernel(const float* __restrict__ in, float* __restrict__ out, int h, int w, int c, int pad_top, int pad_left,
    int h2, int w2, size_t total)
{
    const int run = 2 * c;
    for (size_t o = (size_t)blockIdx.x * blockDim.x + threadIdx.x; o < total; o += (size_t)gridDim.x * blockDim.x) {
        const int dy = (int)(o & 1);
        size_t rest = o >> 1;
        const int x2 = (int)(rest % (size_t)w2);
        rest /= (size_t)w2;
        const int y2 = (int)(rest % (size_t)h2);
        const size_t img = rest / (size_t)h2;
        const int iy = 2 * y2 + dy - pad_top, ix0 = 2 * x2 - pad_left;
        float* dst = out + (o >> 1) * (size_t)(2 * run) + (size_t)dy * run;
        const bool row_ok = iy >= 0 && iy < h;
        const float* src = in + ((img * h + (row_ok ? iy : 0)) * (size_t)w) * c;
        for (int q = 0; q < run; q += 2) { // run = 2c is even and dst is 8-byte aligned: pairs keep the stores whole
            const int ixa = ix0 + q / c, ixb = ix0 + (q + 1) / c;
            float2 v;
            v.x = (row_ok && ixa >= 0 && ixa < w) ? src[(size_t)ixa * c + q % c] : 0.f;
            v.y = (row_ok && ixb >= 0 && ixb < w) ? src[(size_t)ixb * c + (q + 1) % c] : 0.f;
            *reinterpret_cast<float2*>(dst + q) = v;
        }
    }
}

} // namespace fdx

using namespace fdx;

extern "C" int fdx_conv2d_s2d_eligible(int cin, int kh, int kw, int sy, int sx, int dy, int dx, int cout)
{
    const int k8 = (kh + 1) & ~1;
    return cin >= 1 && cin <= 4 && kh == kw && kh >= 2 && sy == 2 && sx == 2 && dy == 1 && dx == 1 && (k8 * 2 * cin) % 16 == 0
        && cout % 4 == 0 && cout >= 64;
}

extern "C" size_t fdx_conv2d_s2d_scratch_bytes(int n, int out_h, int out_w, int cin, int k)
{
    const int k2 = ((k + 1) & ~1) / 2;
    return sizeof(float) * (size_t)n * (size_t)(out_h + k2 - 1) * (size_t)(out_w + k2 - 1) * 4 * (size_t)cin + 256;
}

extern "C" size_t fdx_conv2d_s2d_weight_floats(int cout, int cin, int k)
{
    const int k2 = ((k + 1) & ~1) / 2;
    return (size_t)cout * k2 * k2 * 4 * cin;
}

// host: weights [cout][k][k][cin] -> [cout][ky][kx][(dy, dx, c)] with w2 = w[2 ky + dy][2 kx + dx][c], zero beyond k
extern "C" fdx_status fdx_conv2d_s2d_prepare(const float* weights, int cout, int cin, int k, float* weights_s2d)
{
    FDX_REQUIRE(weights && weights_s2d && cout > 0 && cin > 0 && k > 0, "conv2d_s2d_prepare: bad arguments");
    const int k2 = ((k + 1) & ~1) / 2;
    size_t o = 0;
    for (int n = 0; n < cout; ++n)
        for (int ky = 0; ky < k2; ++ky)
            for (int kx = 0; kx < k2; ++kx)
                for (int dy = 0; dy < 2; ++dy)
                    for (int dx = 0; dx < 2; ++dx)
                        for (int c = 0; c < cin; ++c) {
                            const int fy = 2 * ky + dy, fx = 2 * kx + dx;
                            weights_s2d[o++] = (fy < k && fx < k) ? weights[(((size_t)n * k + fy) * k + fx) * cin + c] : 0.f;
                        }
    return FDX_OK;
}

extern "C" fdx_status fdx_conv2d_s2d_nhwc_f32(const float* in, int n, int h, int w, int cin, const float* weights_s2d,
    const float* bias, int cout, int k, int pad_top, int pad_left, int out_h, int out_w, const float* residual,
    const fdx_act* act, float* scratch, float* out)
{
    FDX_REQUIRE(in && weights_s2d && scratch && out && n > 0 && h > 0 && w > 0 && out_h > 0 && out_w > 0, "conv2d_s2d: bad arguments");
    FDX_REQUIRE(fdx_conv2d_s2d_eligible(cin, k, k, 2, 2, 1, 1, cout), "conv2d_s2d: shape not eligible");
    FDX_REQUIRE(pad_top >= 0 && pad_left >= 0, "conv2d_s2d: negative padding");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    const int k2 = ((k + 1) & ~1) / 2, h2 = out_h + k2 - 1, w2 = out_w + k2 - 1, c4 = 4 * cin;
    FDX_REQUIRE((int64_t)n * h2 * w2 * c4 < (1LL << 29) && (int64_t)n * out_h * out_w < (1LL << 31), "conv2d_s2d: dimension overflow");
    const size_t total = (size_t)n * h2 * w2 * c4, items = (size_t)n * h2 * w2 * 2;
    profile_begin();
    hipLaunchKernelGGL(s2d_kernel, dim3((unsigned)std::min<size_t>((items + 255) / 256, 256 * 32)), dim3(256), 0, stream(), in, scratch, h, w,
        cin, pad_top, pad_left, h2, w2, items);
    profile_end("space_to_depth_f32", 0.0, 4.0 * ((double)n * h * w * cin + (double)total));
    FDX_LAUNCH_CHECK();
    GemmParams p {};
    p.A = scratch; p.B = weights_s2d; p.C = out; p.bias = bias; p.residual = residual;
    p.M = n * out_h * out_w; p.N = cout; p.K = k2 * k2 * c4;
    p.lda = 0; p.ldb = p.K; p.ldc = cout;
    p.alpha = 1.f; p.bias_per_row = 0; p.act = make_act(act);
    p.inner = 1;
    p.H = h2; p.W = w2; p.Cin = k2 * c4; p.pix_stride = c4; p.kh = k2; p.kw = 1; p.sy = 1; p.sx = 1; p.dy = 1; p.dx = 1;
    p.pad_top = 0; p.pad_left = 0; p.OH = out_h; p.OW = out_w;
    // the profile counts the layer's own multiply-adds, not the zero taps of the widened filter
    return run_igemm(p, true, 1, "conv_igemm_f32", 2.0 * p.M * (double)cout * k * k * cin);
}

extern "C" fdx_status fdx_debug_force_tile(int cfg)
{
    fdx::g_forced_tile = cfg;
    return FDX_OK;
}

namespace fdx {
// out[M][n] = act(LN(x)[M][k] . w^T + bias + residual), the rows of x normalised over k inside the GEMM (LNF in
// igemm_fast.hpp): w is the filter with LayerNormalization's gamma folded in ([n][k]), bias the bias with beta folded in,
// wsum[n] the row sums of w.  FDX_ERR_UNSUPPORTED, with nothing launched, where the fast path does not apply.
bool gemm_ln_supported(int64_t m, int n, int k)
{
    return m > 0 && m < (1LL << 31) && n >= 16 && n % 4 == 0 && k >= 32 && k % 32 == 0 && (m * k) * 4 < (1LL << 31);
}

fdx_status gemm_ln_launch(const float* x, int64_t m, int k, const float* w, const float* bias, const float* wsum, float eps, const float* residual,
    const fdx_act* act, float* out, int n)
{
    FDX_REQUIRE(x && w && wsum && out && gemm_ln_supported(m, n, k), "gemm_ln: bad arguments");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    GemmParams p {};
    p.A = x; p.B = w; p.C = out; p.bias = bias; p.residual = residual;
    p.M = (int)m; p.N = n; p.K = k; p.lda = k; p.ldb = k; p.ldc = n;
    p.alpha = 1.f; p.bias_per_row = 0; p.act = make_act(act);
    p.inner = 1;
    p.ln_wsum = wsum;
    p.ln_eps = eps;
    return run_igemm(p, false, 1, "gemm_ln_f32");
}
} // namespace fdx

extern "C" fdx_status fdx_debug_dual_conv(int one_launch)
{
    fdx::g_dual_one_launch = one_launch != 0;
    return FDX_OK;
}

// tests: caps the persistent grid (0 = as many workgroups as are resident on the chip)
extern "C" fdx_status fdx_debug_force_strips(int strips)
{
    FDX_REQUIRE(strips >= 0 && strips <= 64, "debug_force_strips: 0 (the traffic model decides) .. 64");
    fdx::g_forced_strips = strips;
    return FDX_OK;
}

extern "C" fdx_status fdx_debug_persist_cap(int workgroups)
{
    // the tile walk hands every eighth workgroup one eighth of the tiles, so a capped grid keeps at least eight
    fdx::g_persist_scale = workgroups > 0 && workgroups < 8 ? 8 : workgroups;
    return FDX_OK;
}

extern "C" fdx_status fdx_conv2d_nhwc_f32(const float* in, int n, int h, int w, int cin,
    const float* weights, const float* bias, int cout, int kh, int kw,
    int sy, int sx, int dy, int dx, int pad_top, int pad_left, int out_h, int out_w,
    const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && weights && out, "conv2d: null pointer");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(n > 0 && h > 0 && w > 0 && cin > 0 && cout > 0 && kh > 0 && kw > 0, "conv2d: bad shape");
    FDX_REQUIRE(sy > 0 && sx > 0 && dy > 0 && dx > 0 && out_h > 0 && out_w > 0, "conv2d: bad stride/dilation/output");
    FDX_REQUIRE(pad_top >= 0 && pad_left >= 0, "conv2d: negative padding");
    // the last tap of the last output must not start beyond what padding can explain
    FDX_REQUIRE((int64_t)n * out_h * out_w < (1LL << 31) && (int64_t)kh * kw * cin < (1LL << 31)
            && (int64_t)h * w * cin < (1LL << 31),
        "conv2d: dimension overflow");
    GemmParams p {};
    p.A = in; p.B = weights; p.C = out; p.bias = bias; p.residual = residual;
    p.M = n * out_h * out_w; p.N = cout; p.K = kh * kw * cin;
    p.lda = 0; p.ldb = p.K; p.ldc = cout;
    p.alpha = 1.f; p.bias_per_row = 0; p.act = make_act(act);
    p.inner = 1;
    p.H = h; p.W = w; p.Cin = cin; p.kh = kh; p.kw = kw; p.sy = sy; p.sx = sx; p.dy = dy; p.dx = dx;
    p.pad_top = pad_top; p.pad_left = pad_left; p.OH = out_h; p.OW = out_w;
    const bool pointwise = kh == 1 && kw == 1 && sy == 1 && sx == 1 && pad_top == 0 && pad_left == 0
        && out_h == h && out_w == w;
    if (pointwise) { // a 1x1 stride-1 convolution is the plain GEMM [n*h*w][cin] x [cout][cin]^T
        p.lda = cin;
        return run_igemm(p, false, 1, "conv1x1_gemm_f32");
    }
    return run_igemm(p, true, 1, "conv_igemm_f32");
}

namespace fdx {
// Pointwise (1x1, stride 1) convolution whose channel count is a multiple of 4 but not of the 16-float slab of the fast
// path: the filter rows were padded with zero taps to k_padded at load, and the pixels are read as rows of k_padded
// floats that are only cin apart -- the surplus floats belong to the next pixel and meet zero taps (the very last
// pixel's surplus lies beyond the buffer extent, which the loads answer with zeros).  Returns FDX_ERR_UNSUPPORTED,
// with nothing launched, where the fast path does not apply; the caller then uses the unpadded filter.
fdx_status conv1x1_padded_launch(const float* in, int64_t rows, int cin, const float* w_padded, int k_padded, const float* bias,
    int cout, const float* residual, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in && w_padded && out && rows > 0 && rows < (1LL << 31) && cin > 0 && cin % 4 == 0 && k_padded > cin
            && k_padded % 16 == 0 && cout > 0,
        "conv1x1_padded: bad arguments");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    if (cout % 4 != 0 || cout < 64 || !aligned16(in) || !aligned16(w_padded) || !aligned16(out) || (residual && !aligned16(residual))
        || (bias && !aligned16(bias)) || ((rows - 1) * cin + k_padded) * 4 >= (1LL << 31))
        return FDX_ERR_UNSUPPORTED;
    GemmParams p {};
    p.A = in; p.B = w_padded; p.C = out; p.bias = bias; p.residual = residual;
    p.M = (int)rows; p.N = cout; p.K = k_padded; p.lda = cin; p.ldb = k_padded; p.ldc = cout;
    p.alpha = 1.f; p.bias_per_row = 0; p.act = make_act(act);
    p.inner = 1;
    p.a_valid_k = cin;
    return run_igemm(p, false, 1, "conv1x1_gemm_f32", 2.0 * (double)rows * cout * cin);
}
} // namespace fdx

namespace fdx {
// The sum of two pointwise convolutions with one epilogue,
//     out[img][y][x][:] = act(W[:, :c1] . in1[img][y][x][:] + W[:, c1:] . in2[img][y * s2y][x * s2x][:] + bias),
// as one GEMM over the concatenated channels (a residual block whose shortcut branch is a 1x1 convolution, strided or
// not: Add(Conv2D(a), Conv2D(b)) of layers/add_layer.hpp:20-29 over layers/conv_2d_layer.hpp:52-56).  w_cat is
// [cout][c1 + c2].  Where the fast path does not apply the two convolutions run one after the other on the same filter
// array, the second adding to the first's result.
fdx_status conv1x1_dual_launch(const float* in1, int n, int oh, int ow, int c1, const float* in2, int h2, int w2, int c2, int s2y, int s2x,
    const float* w_cat, const float* bias, int cout, const fdx_act* act, float* out)
{
    FDX_REQUIRE(in1 && in2 && w_cat && out && n > 0 && oh > 0 && ow > 0 && c1 > 0 && c2 > 0 && h2 > 0 && w2 > 0 && s2y > 0 && s2x > 0
            && cout > 0 && (int64_t)(oh - 1) * s2y < h2 && (int64_t)(ow - 1) * s2x < w2,
        "conv1x1_dual: bad arguments");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE((int64_t)n * oh * ow < (1LL << 31) && (int64_t)h2 * w2 * c2 < (1LL << 31), "conv1x1_dual: dimension overflow");
    const bool fused = g_dual_one_launch;
    GemmParams p {};
    p.A = in1; p.B = w_cat; p.C = out; p.bias = bias; p.residual = nullptr;
    p.M = n * oh * ow; p.N = cout; p.K = c1 + c2;
    p.lda = c1; p.ldb = p.K; p.ldc = cout;
    p.alpha = 1.f; p.bias_per_row = 0; p.act = make_act(act);
    p.inner = 1;
    p.OH = oh; p.OW = ow;
    p.A2 = in2; p.K1 = c1; p.H2 = h2; p.W2 = w2; p.C2 = c2; p.s2y = s2y; p.s2x = s2x;
    if (fused) {
        const fdx_status st = run_igemm(p, false, 1, "conv1x1_gemm_f32");
        if (st != FDX_ERR_UNSUPPORTED)
            return st;
    }
    // one after the other: the strided one first, without bias and activation, then the other on top of it
    GemmParams a {};
    a.A = in2; a.B = w_cat + c1; a.C = out;
    a.M = p.M; a.N = cout; a.K = c2; a.lda = 0; a.ldb = p.K; a.ldc = cout;
    a.alpha = 1.f; a.act = make_act(nullptr);
    a.inner = 1;
    a.H = h2; a.W = w2; a.Cin = c2; a.kh = 1; a.kw = 1; a.sy = s2y; a.sx = s2x; a.dy = 1; a.dx = 1; a.OH = oh; a.OW = ow;
    fdx_status st;
    if (s2y == 1 && s2x == 1 && h2 == oh && w2 == ow) {
        a.lda = c2;
        st = run_igemm(a, false, 1, "conv1x1_gemm_f32");
    } else {
        st = run_igemm(a, true, 1, "conv_igemm_f32");
    }
    if (st != FDX_OK)
        return st;
    GemmParams b = p;
    b.A2 = nullptr;
    b.K = c1;
    b.residual = out;
    return run_igemm(b, false, 1, "conv1x1_gemm_f32");
}
} // namespace fdx

extern "C" fdx_status fdx_gemm_bias_act_f32(const float* a, int64_t lda, const float* b_nk, int64_t ldb,
    int m, int n, int k, float alpha, const float* bias, int bias_per_row,
    const float* residual, const fdx_act* act, float* c, int64_t ldc, const fdx_gemm_batch* batch)
{
    FDX_REQUIRE(a && b_nk && c, "gemm: null pointer");
    FDX_REQUIRE_EPILOGUE_ACT(act);
    FDX_REQUIRE(m > 0 && n > 0 && k > 0 && lda >= k && ldb >= k && ldc >= n, "gemm: bad shape m=%d n=%d k=%d", m, n, k);
    GemmParams p {};
    p.A = a; p.B = b_nk; p.C = c; p.bias = bias; p.residual = residual;
    p.M = m; p.N = n; p.K = k; p.lda = lda; p.ldb = ldb; p.ldc = ldc;
    p.alpha = alpha; p.bias_per_row = bias_per_row; p.act = make_act(act);
    p.inner = 1;
    int nb = 1;
    if (batch) {
        FDX_REQUIRE(batch->batch > 0 && batch->inner > 0 && batch->batch <= 65535, "gemm: bad batch");
        nb = batch->batch;
        p.inner = batch->inner;
        p.a_outer = batch->a_outer; p.a_inner = batch->a_inner;
        p.b_outer = batch->b_outer; p.b_inner = batch->b_inner;
        p.c_outer = batch->c_outer; p.c_inner = batch->c_inner;
    }
    return run_igemm(p, false, nb, "gemm_f32");
}

// ---- the tuner's table as text: one line per shape, "conv M N K Cin kh kw sy sx batch res choice"
extern "C" fdx_status fdx_tuner_export(char* text, size_t capacity, size_t* needed)
{
    std::string out;
    {
        std::lock_guard<std::mutex> lock(fdx::g_tune_mutex);
        char line[256];
        for (const auto& kv : fdx::g_tuned) {
            const fdx::TuneKey& k = kv.first;
            std::snprintf(line, sizeof line, "%d %d %d %d %d %d %d %d %d %d %d %d\n", k.conv, k.M, k.N, k.K, k.Cin, k.kh, k.kw, k.sy, k.sx,
                k.batch, k.res, kv.second);
            out += line;
        }
    }
    if (needed)
        *needed = out.size() + 1;
    if (text && capacity > 0) {
        FDX_REQUIRE(capacity >= out.size() + 1, "tuner_export: buffer of %zu bytes, %zu needed", capacity, out.size() + 1);
        std::memcpy(text, out.c_str(), out.size() + 1);
    }
    return FDX_OK;
}

extern "C" fdx_status fdx_tuner_import(const char* text)
{
    FDX_REQUIRE(text, "tuner_import: null text");
    std::vector<std::pair<fdx::TuneKey, int>> rows;
    const char* p = text;
    while (*p) {
        fdx::TuneKey k;
        std::memset(&k, 0, sizeof k);
        int choice = 0, used = 0;
        const int got = std::sscanf(p, "%d %d %d %d %d %d %d %d %d %d %d %d%n", &k.conv, &k.M, &k.N, &k.K, &k.Cin, &k.kh, &k.kw, &k.sy,
            &k.sx, &k.batch, &k.res, &choice, &used);
        if (got <= 0)
            break; // trailing white space
        FDX_REQUIRE(got == 12, "tuner_import: malformed line near offset %d", (int)(p - text));
        FDX_REQUIRE(k.conv >= 0 && k.conv <= 3 && choice >= -1, "tuner_import: value out of range near offset %d", (int)(p - text));
        rows.emplace_back(k, choice);
        p += used;
        while (*p == '\n' || *p == '\r' || *p == ' ')
            ++p;
    }
    std::lock_guard<std::mutex> lock(fdx::g_tune_mutex);
    for (const auto& r : rows)
        fdx::g_tuned[r.first] = r.second;
    return FDX_OK;
}

extern "C" fdx_status fdx_tuner_timing(int on)
{
    std::lock_guard<std::mutex> lock(fdx::g_tune_mutex);
    fdx::g_tune_timing = on != 0 ? 1 : 0;
    return FDX_OK;
}

extern "C" fdx_status fdx_tuner_freeze(int on)
{
    std::lock_guard<std::mutex> lock(fdx::g_tune_mutex);
    fdx::g_tune_frozen = on != 0;
    return FDX_OK;
}

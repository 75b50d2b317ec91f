// Launch parameters shared by the implicit-GEMM kernels.
#pragma once
#include <cstring>
#include <functional>
#include "common.hpp"

namespace fdx {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct GemmParams {
    const float* A;
    const float* B;
    float* C;
    const float* bias;
    const float* residual;
    int M, N, K;
    int64_t lda, ldb, ldc;
    float alpha;
    int bias_per_row;
    Act act;
    int inner;
    int64_t a_outer, a_inner, b_outer, b_inner, c_outer, c_inner;
    // convolution view of A
    int H, W, Cin, kh, kw, sy, sx, dy, dx, pad_top, pad_left, OH, OW;
    // fast path: floats between neighbouring input pixels (= Cin, except for the space-to-depth view of a stem
    // convolution, where a filter row reads a run of Cin floats that spans several pixels)
    int pix_stride;
    // fast path only: byte extents of one problem's A (counted from the shifted base) and B operands
    uint32_t a_records, b_records;
    int batch; // number of independent problems folded into the persistent tile walk
    // rows of A that are shorter than K (a pointwise convolution whose channel count was rounded up to the slab with
    // zero filter taps): floats of a row that really exist, 0 = K.  The loads of the last row stop at the real extent.
    int a_valid_k;
    // split-K variant of the fast path: K ranges per tile, partial-tile workspace, one ticket per tile (zero between launches)
    int splits;
    int split_dp_tiles; // leading tiles that are computed whole (one unit each); the rest are cut into `splits` K ranges
    float* split_ws;
    int* split_tickets;
    // fast path, whole-tile launches: output tiles are numbered strip by strip (strip_w column tiles wide, row tiles
    // inside a strip, columns fastest) instead of row by row, so that the contiguous tile range of an XCD needs only
    // its strip's columns of B; 0 = one strip (row by row)
    int strip_w;
    // fast path, GEMM form, whole tiles: a second source of A rows (see DUAL in igemm_fast.hpp); A2 == nullptr = none.
    // K1 = columns taken from A (a multiple of the K slab), the remaining K - K1 come from A2; OH / OW above give the
    // output map the rows are pixels of.
    const float* A2;
    int K1, H2, W2, C2, s2y, s2x;
    uint32_t a2_records;
    // fast path, GEMM form, whole tiles: rows of A layer-normalised over K on the way (see LNF in igemm_fast.hpp);
    // ln_wsum = per output column the sum of its (gamma-folded) filter row, nullptr = no normalisation
    const float* ln_wsum;
    float ln_eps;
};

// Key of the per-process tuning table (igemm.hip).  conv = 0 / 1: a GEMM / convolution shape and its tile choice
// (configuration + 100 * splits + 10000 * mode); conv = 2: a depthwise 3x3 + 1x1 pair (M = height, Cin = width,
// K = channels, N = filters, sy = stride, res = residual, kh = input channels of a whole block) and the form it runs
// in (1 = depthwise + projection as one launch, 2 = a launch per layer, 3 = the whole block as one launch);
// conv = 3: a 3x3 stride-1 convolution (M = output pixels of the batch, kh / kw = input height / width, sy / sx = top /
// left padding) and its kernel (0 = direct, 1 = Winograd).
struct TuneKey {
    int conv, M, N, K, Cin, kh, kw, sy, sx, batch, res;
    bool operator<(const TuneKey& o) const { return std::memcmp(this, &o, sizeof(TuneKey)) < 0; }
};
bool tune_lookup(const TuneKey& key, int* choice);
void tune_store(const TuneKey& key, int choice);
bool tune_frozen(); // fdx_tuner_freeze(1): shapes not in the table take the closed rules, nothing is timed
// The shader clock climbs for about 30 ms after an idle period (2.0 -> 2.4 GHz measured), and candidates timed along the
// climb are not comparable: the later ones look faster.  A timing run that starts after a pause first repeats `launch`
// (rounds of three, a stream synchronisation after each; false from it ends the repetition) for that long; runs that
// follow one another within a few milliseconds, as the shapes of a model's first pass do, find the clock where the one
// before left it.  tune_mark() is called at the end of every timing run.
void tune_settle_clock(const std::function<bool()>& launch);
void tune_mark();

} // namespace fdx

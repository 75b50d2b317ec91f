// Launch parameters of the decode-shape kernels (decode_kernels.hip).
#pragma once
#include "common.hpp"

namespace fdx {

struct SkinnySegment {
    float* ptr;         // output base of this column range
    int64_t ld;         // row stride in floats
    int col_begin;      // first output column stored here
    int64_t len_stride; // if non-zero the base is advanced by *len_dev * len_stride floats (cache rows)
};

struct SkinnyParams {
    const float* X;     // [M][K] activation rows, M <= 16
    int64_t ldx;
    const float* W;     // [N][K], K contiguous (LayerNorm gamma already folded in when ln != 0)
    int64_t ldw;
    int packed;         // W is in the pre-packed tile/wave/slab/lane order written by pack_weights_launch
    int M, N, K;
    const float* bias;  // [N] or null (LayerNorm beta already folded in when ln != 0)
    const float* residual; // [M][N] (row stride ldr) or null
    int64_t ldr;
    Act act;
    int ln;             // rows of X are layer-normalised over K before the product
    float ln_eps;
    const float* w_rowsum; // [N] row sums of the folded W, needed when ln != 0
    int n_seg;
    SkinnySegment seg[3];
    const int* len_dev; // device int read by segments with len_stride != 0
    // optional split-K support: partial tiles [split][tile][256] and one zero-initialised ticket per tile
    float* workspace;
    int64_t workspace_floats;
    int* tickets;
    int ticket_count;
    // optional, wide-output launches only (skinny_wide_grid(p) > 0): every workgroup leaves the packed (value, column)
    // maximum of each row over the columns it produced in amax_parts[workgroup][16]; argmax_parts_launch picks the winner
    unsigned long long* amax_parts;
};

fdx_status skinny_gemm_launch(const SkinnyParams& p);

// One phase of the persistent decode-step kernel: a Dense launch (as skinny_gemm_launch would run it) or the decode
// attention of every (sequence, head).
struct MegaPhase {
    int kind;    // 0 = Dense, 1 = attention
    int tiles;   // Dense: 16-column groups; attention: (sequence, head) items
    int ksplit;  // Dense: K ranges per column group
    int chunk;   // Dense: 6 or 8 slabs per wave (the kernel instantiation)
    SkinnyParams g;
    const float* q;
    int64_t ldq;
    const float* kc;
    const float* vc;
    float* out;
    int heads, max_len;
    float scale;
};
// Fills `phase` from a Dense launch's parameters; false when the persistent kernel does not cover the shape.
bool mega_dense_phase(const SkinnyParams& p, float* workspace, int* tickets, MegaPhase& phase);
bool mega_attention_phase(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch, int heads, int dk,
    int dv, const int* len_dev, int max_len, MegaPhase& phase);
// Device-side state of the persistent kernel's grid barrier (allocated once per session): arrival cells, release cells,
// epoch, abort flag.
size_t mega_state_bytes();
// Runs the phases back to back inside one launch, a grid-wide barrier between consecutive phases.
fdx_status mega_launch(const MegaPhase* phases_dev, int n_phases, void* state_dev);
// non-zero after a launch whose barrier gave up waiting (reads the flag back; synchronises the stream)
fdx_status mega_check(void* state_dev);
// number of workgroups the launch would use if it takes the wide-output kernel (one that strides over column groups), else 0
int skinny_wide_grid(const SkinnyParams& p);
// greedy ids from per-workgroup partial maxima [parts][16] (first maximum wins), then as argmax_bump_launch
fdx_status argmax_parts_launch(const unsigned long long* amax_parts, int parts, int rows, float* out_idx_f, int* len_dev, float* history);
fdx_status skinny_prepare();
int64_t packed_weight_floats(int n, int k);
fdx_status pack_weights_launch(const float* w, int n, int k, int64_t ldw, float* out);
fdx_status fold_layernorm_launch(const float* gamma, const float* beta, const float* w, const float* bias, int n, int k,
    float* w_out, float* wsum, float* bias_out);
fdx_status embed_add_launch(const float* ids, int batch, const float* ta, int dim_a, const float* tb, int dim_b,
    const int* len_dev, int depth, float* out, int* err, unsigned long long* amax);
fdx_status mha_decode_dyn_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch,
    int heads, int dk, int dv, const int* len_dev, int max_len, int len_hint);
fdx_status argmax_bump_launch(const float* x, int rows, int depth, float* out_idx_f, int* len_dev, unsigned long long* amax,
    float* history);
fdx_status set_int_launch(int* p, int v);

} // namespace fdx

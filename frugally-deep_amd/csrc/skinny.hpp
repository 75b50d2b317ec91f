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
    // The K ranges of a column group exchange their partial tiles inside their XCD's L2 instead of through memory:
    // with a number of column groups that is a multiple of 8 the workgroups (bx, 0..splits-1) all run on XCD bx % 8
    // (workgroups go round the XCDs by their linear index).  The last K range of a group waits, bounded, for flags the
    // others store next to the tickets (tickets[ticket_count / 2 + bx * 8 + split], zero between launches), adds the
    // partials in split order and runs the epilogue.  err (may be null) receives kErrSplitExchange if a wait runs out or
    // the flags name another XCD.
    int local_split;
    int* err;
    // Optional: with emb_x != 0 the activation rows are not read from X but formed on the way in as the sum of two
    // embedding rows, row i = emb_a[(int)emb_ids[i]][:] + emb_b[*len_dev][:] (token + position embedding of the token a
    // decode step starts from, layers/embedding_layer.hpp:38-58 twice and an Add); with emb_res != 0 the residual operand
    // is that sum (residual is then ignored; the tables' depth must equal N).  An id outside [0, emb_a_rows) or a position outside [0, emb_b_rows) sets *emb_err to 1
    // and contributes zeros.  Not with the wide-output kernel and not with K split across workgroups.
    const float* emb_ids;
    const float* emb_a;
    const float* emb_b;
    int emb_a_rows, emb_b_rows;
    int emb_x, emb_res;
    int* emb_err;
    // optional, wide-output launches only (skinny_wide_grid(p) > 0): every workgroup leaves the packed (value, column)
    // maximum of each row over the columns it produced in amax_parts[workgroup][16]; argmax_parts_launch picks the winner
    unsigned long long* amax_parts;
};

constexpr int kErrSplitExchange = 2; // value of the err cell: the partial tiles of a split launch did not meet

fdx_status skinny_gemm_launch(const SkinnyParams& p);

// number of workgroups the launch would use if it takes the wide-output kernel (one that strides over column groups), else 0
int skinny_wide_grid(const SkinnyParams& p);
// greedy ids from per-workgroup partial maxima [parts][16] (first maximum wins), then as argmax_bump_launch
fdx_status argmax_parts_launch(const unsigned long long* amax_parts, int parts, int rows, float* out_idx_f, int* len_dev, float* history);
// ... and the token + position embedding of the picked ids at the position they take, into x0 (the next step's first launch)
fdx_status argmax_parts_embed_launch(const unsigned long long* amax_parts, int parts, int rows, float* out_idx_f, int* len_dev, float* history,
    const float* ta, int dim_a, const float* tb, int dim_b, int depth, float* x0, int* err);
fdx_status skinny_prepare();
int64_t packed_weight_floats(int n, int k);
fdx_status pack_weights_launch(const float* w, int n, int k, int64_t ldw, float* out);
fdx_status fold_layernorm_launch(const float* gamma, const float* beta, const float* w, const float* bias, int n, int k,
    float* w_out, float* wsum, float* bias_out);
fdx_status embed_add_launch(const float* ids, int batch, const float* ta, int dim_a, const float* tb, int dim_b,
    const int* len_dev, int depth, float* out, int* err, unsigned long long* amax);
// Decode attention (64-wide heads, at most 256 cached positions) and the layer's output projection with bias, residual and
// activation as one launch (decode_attn.hip); wt is the projection kernel re-laid by pack_proj_heads_launch, workspace
// holds batch * heads * n_out partial sums, tickets one zero-initialised cell per sequence.
bool mha_decode_proj_supported(int batch, int heads, int dk, int dv, int max_len, int64_t ldq, int n_out, int64_t workspace_floats,
    int ticket_count);
fdx_status pack_proj_heads_launch(const float* w_nk, int heads, int n_out, float* out);
fdx_status mha_decode_proj_launch(const float* q, int64_t ldq, const float* kc, const float* vc, int batch, int heads,
    const int* len_dev, int max_len, const float* wt, const float* bias, const float* residual, int64_t ldr, const Act& act, int n_out,
    float* workspace, int64_t workspace_floats, int* tickets, int ticket_count, float* out, int len_hint);
fdx_status mha_decode_dyn_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch,
    int heads, int dk, int dv, const int* len_dev, int max_len, int len_hint);
fdx_status argmax_bump_launch(const float* x, int rows, int depth, float* out_idx_f, int* len_dev, unsigned long long* amax,
    float* history);
fdx_status set_int_launch(int* p, int v);

} // namespace fdx

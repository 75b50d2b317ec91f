// In-memory form of a loaded model: a flat list of device ops (after load-time fusion),
// resident weights, and per-input-shape launch plans.
#pragma once
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "common.hpp"
#include "einsum.hpp"

namespace fdx {

enum class OpKind {
    Input, Conv2D, DWConv2D, Dense, Affine, LayerNorm, Act, Softmax, ZeroPad, Pool, GlobalPool, Add, Embedding, MHA, View, Einsum, Concat, Host, PReLU, Resize, Crop, Permute, Dilate
};

using Shape = std::vector<int64_t>; // dims of one sample, no batch axis

inline int64_t volume(const Shape& s)
{
    int64_t v = 1;
    for (auto d : s)
        v *= d;
    return v;
}

struct Op {
    OpKind kind = OpKind::View;
    std::string name, cls;
    std::vector<int> in; // producer op indices
    int residual = -1;   // op whose output is added in the producer's epilogue
    int fuse_dw = -1;    // 1x1 Conv2D: the depthwise 3x3 op in front of it that one launch can absorb (fdx_dwconv_pointwise_nhwc_f32)
    int fused_into = -1; // that depthwise op: the convolution which may absorb it
    int fuse_exp = -1;   // 1x1 Conv2D with fuse_dw >= 0: the 1x1 expansion in front of the depthwise op, if one launch can run all three (fdx_inverted_residual_nhwc_f32)
    int exp_into = -1;   // that expansion: the projection which may absorb it
    // 1x1 stride-1 Conv2D that has absorbed the 1x1 convolution of its residual operand (conv1x1_dual_launch): input
    // channels and strides of that convolution, whose input is in[1]; the filter over both inputs' channels is weight
    // array 5
    int dual_cin = 0, dual_sy = 1, dual_sx = 1;
    // 1x1 stride-1 Conv2D whose result feeds another one (the tail of a residual block and the convolution that opens the
    // next block): chain = that consumer, chained_from on the consumer = this op.  Where a plan runs the pair as one launch
    // (conv1x1_chain_launch) the consumer's result is produced here and its own turn is skipped; the packed filters are
    // weight array 6 of both ops.
    int chain = -1, chained_from = -1;
    // Dense / self-attention op whose input is a LayerNormalization over the last axis that feeds nothing else but such
    // ops: ln_src = that op, ln_eps its epsilon.  Where a plan normalises inside the GEMM (gemm_ln_launch) the op reads the
    // LayerNormalization's own input and the weight arrays with gamma / beta folded in (Dense: arrays 2-4 = filter, bias,
    // filter row sums; attention: arrays 12-14, the same for the stacked query / key / value projection), and the
    // LayerNormalization launch is skipped.
    int ln_src = -1;
    float ln_eps = 0.f;
    bool dead = false;
    int consumers = 0;

    // attributes
    int cout = 0, kh = 1, kw = 1, sy = 1, sx = 1, dy = 1, dx = 1, padding = 0;
    int zp[4] = { 0, 0, 0, 0 }; // folded explicit zero padding: top, bottom, left, right
    Act act { FDX_ACT_NONE, 3.402823466e+38f, 0.f, 0.f };
    bool softmax = false; // fused "softmax" activation runs as a second kernel
    int pool_mode = 0;
    bool keepdims = false;
    float eps = 0.f;
    int ln_axes = 1;
    int heads = 0, dk = 0, dv = 0, dout = 0, d_in = 0;
    bool use_bias = true;
    int input_dim = 0, output_dim = 0, units = 0, n_in = 0;
    Shape target_shape;
    bool flatten = false;
    int input_index = -1;
    std::string equation, bias_axes; // EinsumDense
    Shape kernel_dims, full_out;     // EinsumDense: kernel extents as stored, output_shape with the batch slot
    bool gemm = false;               // EinsumDense that is one row-major GEMM (kernel stored transposed)
    int axis = -1;                   // Concatenate
    int host_index = -1;             // Host: index into fdx_model::host_layers
    int combine = 0;                 // Add-like merges: FDX_COMBINE_* operation
    float scale = 1.0f;              // Average: 1 / number of inputs
    bool log_after = false;          // Softmax op that is a log_softmax
    bool rms = false;                // LayerNorm op that is an RMSNormalization
    bool bilinear = false;           // Resize: interpolation (kh / kw hold the factors; Crop keeps its margins in zp)
    bool affine_scalar = false;      // Affine with one (scale, shift) pair for the whole tensor (Rescaling, axis-less Normalization)
    bool trailing = false;           // Dilate: zero insertion in front of a "same" transposed convolution (kh / kw hold the rates)
    bool gate = false;               // attention with a sigmoid gate on its output (GroupQueryAttention use_gate)
    std::vector<int64_t> shared_axes; // PReLU

    // host weights (released after upload)
    std::vector<std::vector<float>> hw;
    // device weights, indexed like hw
    std::vector<float*> dw;
};

struct Block {
    void* p = nullptr;
    size_t bytes = 0;
    bool busy = false;
};

struct Plan {
    int batch = 0;
    std::vector<Shape> in_shapes;
    std::vector<Shape> shapes;   // per op
    std::vector<float*> out;     // per op output buffer (device)
    std::vector<int> order;      // execution order (live ops)
    std::vector<int> block_of;   // per op: index into blocks, -1 = alias / external
    std::vector<int> last_use;   // position in order of the last consumer
    std::vector<Block> blocks;
    std::vector<std::vector<float*>> temps; // per op: scratch placed at plan time
    std::vector<signed char> dw_fused;      // per 1x1 convolution with fuse_dw >= 0: 0 = not timed yet, 1 = depthwise + projection as one launch, 2 = one launch per layer, 3 = expansion + depthwise + projection as one launch
    std::vector<signed char> conv_form;     // per 3x3 stride-1 convolution with a Winograd filter: -1 = not timed yet, 0 = direct kernel, 1 = Winograd kernel
    std::vector<signed char> chain_on;      // per 1x1 convolution with chain >= 0: 1 = this plan runs it and its consumer as one launch
    std::vector<signed char> ln_fold_on;    // per Dense / attention op with ln_src >= 0: 1 = this plan normalises inside its GEMM
    std::vector<signed char> ln_skip;       // per LayerNormalization op: 1 = every reader normalises for itself, no launch
    std::vector<signed char> chain_done;    // per consumer of such a pair: its result was produced by the producer's launch in this run
    double flops = 0;
    ~Plan();
};

} // namespace fdx

// one custom layer object created through fdx_custom_layer::create
struct fdx_host_layer {
    fdx_custom_layer vt;
    void* instance = nullptr;
};

struct fdx_model {
    std::string name, hash;
    std::vector<fdx_host_layer> host_layers;
    std::vector<fdx::Op> ops;
    std::vector<int> inputs, outputs;   // op indices
    std::vector<fdx::Shape> in_decl, out_decl; // declared shapes, -1 = variable
    std::vector<float*> device_allocs;
    int* err_flag = nullptr;
    bool has_embedding = false;
    // launch plans keyed by (batch, per-sample input shapes), most recently used first; a model fed alternating shapes
    // (variable input dimensions, tensor_shape_variable.hpp) keeps up to kMaxPlans of them instead of re-planning
    static constexpr size_t kMaxPlans = 4;
    std::vector<std::unique_ptr<fdx::Plan>> plans;
    std::mutex mu;
    double last_flops = 0;
    ~fdx_model();
};

namespace fdx {
// builds (or reuses) the plan for this batch and these per-sample input shapes
fdx_status get_plan(fdx_model* m, int batch, const std::vector<Shape>& in_shapes, Plan** out);
float* plan_alloc(Plan& p, size_t bytes, int* block_index);
std::vector<int> topo_order(const fdx_model& m); // producers before consumers, dead ops skipped by callers
fdx_status positions_launch(float* out, int batch, int t, int start);
bool chain_supported(int k1, int k2, int n1, int n2);
size_t chain_first_floats(int n1, int k);
size_t chain_second_floats(int n1, int n2);
void chain_pack_first(const float* w, int n1, int k, float* out);
void chain_pack_second(const float* w, int n1, int n2, float* out);
fdx_status conv1x1_chain_launch(const float* a, int n, int oh, int ow, int k1, const float* b, int h2, int w2, int c2, int s2y, int s2x,
    int k2, const float* w1, const float* bias1, const float* residual, const fdx_act* act1, int n1, float* y, const float* w2p,
    const float* bias2, const fdx_act* act2, int n2, float* z);
bool gemm_ln_supported(int64_t m, int n, int k);
fdx_status gemm_ln_launch(const float* x, int64_t m, int k, const float* w, const float* bias, const float* wsum, float eps, const float* residual,
    const fdx_act* act, float* out, int n);
fdx_status conv1x1_dual_launch(const float* in1, int n, int oh, int ow, int c1, const float* in2, int h2, int w2, int c2, int s2y, int s2x,
    const float* w_cat, const float* bias, int cout, const fdx_act* act, float* out);
fdx_status conv1x1_padded_launch(const float* in, int64_t rows, int cin, const float* w_padded, int k_padded, const float* bias,
    int cout, const float* residual, const fdx_act* act, float* out);
fdx_status mha_prefill_strided(const float* q, int64_t ldq, int64_t q_batch, const float* k, int64_t ldk, int64_t k_batch,
    const float* v, int64_t ldv, int64_t v_batch, int batch, int t, int s, int heads, int dk, int dv, int causal,
    float* out, int64_t ldo, int64_t o_batch, void* scratch_dev);
fdx_status argmax_launch(const float* x, int64_t rows, int depth, int32_t* out_idx, float* out_val, float* out_idx_f);
fdx_status einsum_launch(EinsumSpec& spec, const float* in, const float* kernel, const float* bias, const Act& act, float* out);
fdx_status gather_rows_launch(const float* in, int64_t rows, int depth, int64_t row_stride, int64_t offset, float* out);
}
